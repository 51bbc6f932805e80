// Paged attention, plain form: one wave per (token, query head), every product and sum in float.
// It is the 32-bit path and the fallback for shapes the MFMA kernels refuse.
//
// Contract (shared by every attention kernel here): token t belongs to request seg[t] and sits at
// absolute position pos[t]; it sees the keys of its request at positions [lo, pos[t]] with
// lo = max(0, pos[t] - window + 1) when window > 0, else 0.  Keys and values are read from the
// paged cache (keys [pages, nkv, page, d], values transposed [pages, nkv, d, page]) through block_tables[seg[t], key / page]; the step has
// already written this step's keys there.
//
// Keys are consumed in chunks of AB_CHUNK keys aligned to absolute key index, and inside a chunk in
// tiles of 64: every chunk gives a partial result (maximum, sum, unnormalised output) from a fresh
// start, and the chunks' partial results are folded in ascending order.  So the order of every
// sum is fixed by (request, position) alone: cutting a prompt into portions or batching it with
// other requests cannot change a bit of the result.  Two launch shapes compute the same bits: one
// wave walks all chunks of its (token, head) and folds as it goes (many tokens: portions of
// prompts), or one wave a chunk writes its partial result to a workspace and a second kernel
// folds them with the same function in the same order (few tokens over long contexts: decoding,
// where one wave a head would leave most of the chip idle).
#include "common.h"

#define AB_CHUNK 512

// (M, L, ACC) <- fold of (M, L, ACC) and a chunk's (m, l, acc); explicit multiply-adds, so that the two
// launch shapes round alike
__device__ __forceinline__ void ab_fold(float& M, float& L, float (&ACC)[4], float m, float l, const float (&acc)[4]) {
    const float Mn = fmaxf(M, m);
    const float a = expf(M - Mn), b = expf(m - Mn);
    L = fmaf(L, a, l * b);
#pragma unroll
    for (int i = 0; i < 4; ++i) ACC[i] = fmaf(ACC[i], a, acc[i] * b);
    M = Mn;
}

// four consecutive elements as floats (p 16 bytes aligned for float, 8 for bfloat16)
__device__ __forceinline__ void load4(const float* p, float* v) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16* p, float* v) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}

#define AB_ONE_KEY(J_)                                                                         \
    {                                                                                          \
        const int key = (tile << 6) + (J_);                                                    \
        const int pg = bt[key / page];                                                         \
        const T* vcol = vc + ((size_t)pg * nkv + kvh) * d * page + (key % page);               \
        const float w = ps[J_];                                                                \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                        \
            const int dim = lane + 64 * i;                                                     \
            if (dim < d) acc[i] = fmaf(w, to_f32(vcol[(size_t)dim * page]), acc[i]);           \
        }                                                                                      \
    }

// VEC: the head size and the page size are multiples of 4 and the tensors 16 bytes aligned: 16-byte loads.
// ws == nullptr: gridDim.z == 1, the wave walks all chunks.  Else blockIdx.z is the chunk (absolute
// index) and the partial result goes to ws[((t * nh + h) * gridDim.z + chunk) * (d + 2)]: d outputs, m, l.
template <typename T, bool VEC>
__global__ void __launch_bounds__(64)
attn_basic_kernel(T* __restrict__ out, float* __restrict__ ws, const T* __restrict__ q, const T* __restrict__ kc,
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
    int c_first = lo / AB_CHUNK, c_last = p / AB_CHUNK;
    if (ws != nullptr) {
        if ((int)blockIdx.z < c_first || (int)blockIdx.z > c_last) return;   // the fold reads only the chunks the token sees
        c_first = c_last = blockIdx.z;
    }
    const int* bt = block_tables + (size_t)seg[t] * max_blocks;
    const T* qrow = q + (size_t)t * q_stride + (size_t)h * d;
    for (int i = lane; i < d; i += 64) qs[i] = to_f32(qrow[i]);
    __syncthreads();

    float M = -INFINITY, L = 0.f;
    float ACC[4] = {0.f, 0.f, 0.f, 0.f};
    for (int c = c_first; c <= c_last; ++c) {
        const int k_lo = lo > c * AB_CHUNK ? lo : c * AB_CHUNK;
        const int k_hi = p < c * AB_CHUNK + AB_CHUNK - 1 ? p : c * AB_CHUNK + AB_CHUNK - 1;
        float m = -INFINITY, l = 0.f;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int tile = k_lo >> 6; tile <= (k_hi >> 6); ++tile) {
            const int kidx = (tile << 6) + lane;
            const bool valid = kidx >= k_lo && kidx <= k_hi;
            float s = -INFINITY;
            if (valid) {
                const int pg = bt[kidx / page];
                const T* krow = kc + (((size_t)pg * nkv + kvh) * page + (kidx % page)) * d;
                float dot = 0.f;
                if (VEC) {   // four dims a load; the sum keeps its ascending order
                    for (int i = 0; i < d; i += 4) {
                        float kv[4];
                        load4(krow + i, kv);
#pragma unroll
                        for (int e = 0; e < 4; ++e) dot = fmaf(qs[i + e], kv[e], dot);
                    }
                } else {
                    for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_f32(krow[i]), dot);
                }
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
            const int j0 = (k_lo > (tile << 6)) ? k_lo - (tile << 6) : 0;
            const int j1 = (k_hi - (tile << 6) < 63) ? k_hi - (tile << 6) : 63;
            int j = j0;
            if (VEC) {
                // four keys a load where they lie in one page, 16 bytes aligned (the page size is a multiple of
                // 4 and tiles begin at multiples of 64): the sum keeps its ascending order
                for (; j <= j1 && (j & 3); ++j) AB_ONE_KEY(j)
                for (; j + 3 <= j1; j += 4) {
                    const int key = (tile << 6) + j;
                    const int pg = bt[key / page];
                    const T* vcol = vc + ((size_t)pg * nkv + kvh) * d * page + (key % page);
                    const float w0 = ps[j], w1 = ps[j + 1], w2 = ps[j + 2], w3 = ps[j + 3];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int dim = lane + 64 * i;
                        if (dim < d) {
                            float vv[4];
                            load4(vcol + (size_t)dim * page, vv);
                            acc[i] = fmaf(w0, vv[0], acc[i]);
                            acc[i] = fmaf(w1, vv[1], acc[i]);
                            acc[i] = fmaf(w2, vv[2], acc[i]);
                            acc[i] = fmaf(w3, vv[3], acc[i]);
                        }
                    }
                }
            }
            for (; j <= j1; ++j) AB_ONE_KEY(j)
            __syncthreads();
            m = m_new;
        }
        if (ws != nullptr) {
            float* dst = ws + (((size_t)t * nh + h) * gridDim.z + c) * (d + 2);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dim = lane + 64 * i;
                if (dim < d) dst[dim] = acc[i];
            }
            if (lane == 0) {
                dst[d] = m;
                dst[d + 1] = l;
            }
            return;
        }
        ab_fold(M, L, ACC, m, l, acc);
    }
    T* orow = out + (size_t)t * out_stride + (size_t)h * d;
    const float inv = 1.0f / L;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int dim = lane + 64 * i;
        if (dim < d) orow[dim] = from_f32<T>(ACC[i] * inv);
    }
}

// Folds the chunks' partial results of one (token, head), in ascending order, as the one-wave shape does.
template <typename T>
__global__ void __launch_bounds__(64)
attn_basic_fold_kernel(T* __restrict__ out, const float* __restrict__ ws, const int* __restrict__ pos, int nh, int d,
                       int nchunks, int out_stride, int window) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    if (p / AB_CHUNK > nchunks - 1) {
        // the caller's bound on the lengths was too small for this token: its last chunks were never computed.
        // A row of NaNs instead of a silently wrong one.
        T* bad = out + (size_t)t * out_stride + (size_t)h * d;
        for (int dim = lane; dim < d; dim += 64) bad[dim] = from_f32<T>(__int_as_float(0x7fc00000));
        return;
    }
    float M = -INFINITY, L = 0.f;
    float ACC[4] = {0.f, 0.f, 0.f, 0.f};
    for (int c = lo / AB_CHUNK; c <= p / AB_CHUNK; ++c) {
        const float* src = ws + (((size_t)t * nh + h) * nchunks + c) * (d + 2);
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int dim = lane + 64 * i;
            if (dim < d) acc[i] = src[dim];
        }
        ab_fold(M, L, ACC, src[d], src[d + 1], acc);
    }
    T* orow = out + (size_t)t * out_stride + (size_t)h * d;
    const float inv = 1.0f / L;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int dim = lane + 64 * i;
        if (dim < d) orow[dim] = from_f32<T>(ACC[i] * inv);
    }
}

extern "C" int ilm_attn_basic_chunk() { return AB_CHUNK; }

// ws: null (one wave walks all chunks of its token and head), or float [T][nh][nchunks][d + 2] with
// nchunks >= ceil((largest position + 1) / ilm_attn_basic_chunk()): one wave a chunk, then the fold.
extern "C" int ilm_attn_basic(void* out, void* ws, int nchunks, const void* q, const void* kc, const void* vc,
                              const void* block_tables, const void* seg, const void* pos, int T_,
                              int nh, int nkv, int d, int page, int max_blocks, int q_stride,
                              int out_stride, float scale, int window, int dtype,
                              hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv > 0 && d > 0 && page > 0 && max_blocks > 0, "attn_basic: bad sizes");
    ILM_REQUIRE(nh % nkv == 0, "attn_basic: %d query heads do not divide into %d groups", nh, nkv);
    ILM_REQUIRE(d <= 256, "attn_basic: head size %d above 256", d);
    ILM_REQUIRE(nh <= 65535, "attn_basic: too many heads");
    ILM_REQUIRE(ws == nullptr || (nchunks >= 1 && nchunks <= 65535), "attn_basic: %d chunks", nchunks);
    ILM_REQUIRE(dtype == ILM_DTYPE_F32 || dtype == ILM_DTYPE_BF16, "attn_basic: unknown dtype %d", dtype);
    dim3 grid(T_, nh, ws != nullptr ? nchunks : 1);
    const size_t shm = (size_t)(d + 64) * sizeof(float);
    const bool vec = d % 4 == 0 && page % 4 == 0 && ((uintptr_t)kc & 15) == 0 && ((uintptr_t)vc & 15) == 0;
#define AB_LAUNCH(T_, VEC_)                                                                                             \
    attn_basic_kernel<T_, VEC_><<<grid, 64, shm, stream>>>(                                                             \
        (T_*)out, (float*)ws, (const T_*)q, (const T_*)kc, (const T_*)vc, (const int*)block_tables, (const int*)seg,    \
        (const int*)pos, nh, nkv, d, page, max_blocks, q_stride, out_stride, scale, window)
    if (dtype == ILM_DTYPE_F32) {
        if (vec) AB_LAUNCH(float, true); else AB_LAUNCH(float, false);
    } else {
        if (vec) AB_LAUNCH(bf16, true); else AB_LAUNCH(bf16, false);
    }
#undef AB_LAUNCH
    ILM_LAUNCH_CHECK("attn_basic");
    if (ws != nullptr) {
        dim3 g2(T_, nh);
        if (dtype == ILM_DTYPE_F32)
            attn_basic_fold_kernel<float><<<g2, 64, 0, stream>>>((float*)out, (const float*)ws, (const int*)pos, nh, d, nchunks,
                                                                 out_stride, window);
        else
            attn_basic_fold_kernel<bf16><<<g2, 64, 0, stream>>>((bf16*)out, (const float*)ws, (const int*)pos, nh, d, nchunks,
                                                                out_stride, window);
        ILM_LAUNCH_CHECK("attn_basic_fold");
    }
    return 0;
}
