// Paged attention, plain form: one wave per (token, query head), every product and sum in float.
// It is the 32-bit path and the fallback for shapes the MFMA kernels refuse.
//
// Contract (shared by every attention kernel here): token t belongs to request seg[t] and sits at
// absolute position pos[t]; it sees the keys of its request at positions [lo, pos[t]] with
// lo = max(0, pos[t] - window + 1) when window > 0, else 0.  Keys and values are read from the
// paged cache (keys [pages, nkv, page, d], values transposed [pages, nkv, d, page]) through block_tables[seg[t], key / page]; the step has
// already written this step's keys there.  Keys are consumed in tiles of 64 aligned to absolute
// key index, so the order of every sum is fixed by (request, position) alone: cutting a prompt
// into portions or batching it with other requests cannot change a bit of the result.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(64)
attn_basic_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc,
                  const T* __restrict__ vc, const int* __restrict__ block_tables,
                  const int* __restrict__ seg, const int* __restrict__ pos, int nh, int nkv, int d,
                  int page, int max_blocks, int q_stride, int out_stride, float scale, int window) {
    extern __shared__ float smem[];
    float* qs = smem;      // d
    float* ps = smem + d;  // 64
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (nh / nkv);
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* bt = block_tables + (size_t)seg[t] * max_blocks;
    const T* qrow = q + (size_t)t * q_stride + (size_t)h * d;
    for (int i = lane; i < d; i += 64) qs[i] = to_f32(qrow[i]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int tile = lo >> 6; tile <= (p >> 6); ++tile) {
        const int kidx = (tile << 6) + lane;
        const bool valid = kidx >= lo && kidx <= p;
        float s = -INFINITY;
        if (valid) {
            const int pg = bt[kidx / page];
            const T* krow = kc + (((size_t)pg * nkv + kvh) * page + (kidx % page)) * d;
            float dot = 0.f;
            for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_f32(krow[i]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float pj = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);
        l = l * corr + wave_sum(pj);
        ps[lane] = pj;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] *= corr;
        const int j0 = (lo > (tile << 6)) ? lo - (tile << 6) : 0;
        const int j1 = (p - (tile << 6) < 63) ? p - (tile << 6) : 63;
        for (int j = j0; j <= j1; ++j) {
            const int key = (tile << 6) + j;
            const int pg = bt[key / page];
            const T* vcol = vc + ((size_t)pg * nkv + kvh) * d * page + (key % page);
            const float w = ps[j];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dim = lane + 64 * i;
                if (dim < d) acc[i] = fmaf(w, to_f32(vcol[(size_t)dim * page]), acc[i]);
            }
        }
        __syncthreads();
        m = m_new;
    }
    T* orow = out + (size_t)t * out_stride + (size_t)h * d;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int dim = lane + 64 * i;
        if (dim < d) orow[dim] = from_f32<T>(acc[i] * inv);
    }
}

extern "C" int ilm_attn_basic(void* out, const void* q, const void* kc, const void* vc,
                              const void* block_tables, const void* seg, const void* pos, int T_,
                              int nh, int nkv, int d, int page, int max_blocks, int q_stride,
                              int out_stride, float scale, int window, int dtype,
                              hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv > 0 && d > 0 && page > 0 && max_blocks > 0, "attn_basic: bad sizes");
    ILM_REQUIRE(nh % nkv == 0, "attn_basic: %d query heads do not divide into %d groups", nh, nkv);
    ILM_REQUIRE(d <= 256, "attn_basic: head size %d above 256", d);
    ILM_REQUIRE(nh <= 65535, "attn_basic: too many heads");
    dim3 grid(T_, nh);
    const size_t shm = (size_t)(d + 64) * sizeof(float);
    if (dtype == ILM_DTYPE_F32)
        attn_basic_kernel<float><<<grid, 64, shm, stream>>>(
            (float*)out, (const float*)q, (const float*)kc, (const float*)vc, (const int*)block_tables,
            (const int*)seg, (const int*)pos, nh, nkv, d, page, max_blocks, q_stride, out_stride, scale, window);
    else if (dtype == ILM_DTYPE_BF16)
        attn_basic_kernel<bf16><<<grid, 64, shm, stream>>>(
            (bf16*)out, (const bf16*)q, (const bf16*)kc, (const bf16*)vc, (const int*)block_tables,
            (const int*)seg, (const int*)pos, nh, nkv, d, page, max_blocks, q_stride, out_stride, scale, window);
    else
        ILM_REQUIRE(false, "attn_basic: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("attn_basic");
    return 0;
}
