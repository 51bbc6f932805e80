// Memory-bound kernels of the step: embedding gather, residual add + RMSNorm, rotation + cache
// write, SwiGLU, row gather.  All arithmetic is float; T is the activation type (float or bf16).
#include <stdarg.h>

#include "common.h"
#include "frag.h"

static thread_local char g_err[1024] = {0};

extern "C" const char* ilm_last_error() { return g_err; }

void ilm_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int ilm_num_cus() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) n = prop.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

// ------------------------------------------------------------------------------------------
// embedding: r[t, :] = scale * E[ids[t], :]   (residual stream, float)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(float* __restrict__ r, const int* __restrict__ ids,
                             const T* __restrict__ table, int H, float scale) {
    const int t = blockIdx.x;
    const T* row = table + (size_t)ids[t] * H;
    float* out = r + (size_t)t * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) out[j] = scale * to_f32(row[j]);
}

extern "C" int ilm_embed(void* r, const void* ids, const void* table, int T_, int H, int V,
                         float scale, int dtype, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T_, H, V);
    if (dtype == ILM_DTYPE_F32)
        embed_kernel<float><<<T_, 256, 0, stream>>>((float*)r, (const int*)ids, (const float*)table, H, scale);
    else if (dtype == ILM_DTYPE_BF16)
        embed_kernel<bf16><<<T_, 256, 0, stream>>>((float*)r, (const int*)ids, (const bf16*)table, H, scale);
    else
        ILM_REQUIRE(false, "embed: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("embed");
    return 0;
}

// eight consecutive elements as floats (16-byte accesses; p must be 16-byte aligned)
template <typename T>
__device__ __forceinline__ void load8(const T* p, float* v) {
    T t[8];
    if (sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(t) = *reinterpret_cast<const uint4*>(p);
    } else {
        *reinterpret_cast<float4*>(t) = *reinterpret_cast<const float4*>(p);
        *reinterpret_cast<float4*>(t + 4) = *reinterpret_cast<const float4*>(p + 4);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_f32(t[e]);
}

// ------------------------------------------------------------------------------------------
// r += alpha * h ; x = r / sqrt(mean(r^2) + eps) * w
// One block per row.  The sum of squares is reduced in an order that depends on H only, so a
// row's result does not depend on what else is in the batch.
// ------------------------------------------------------------------------------------------
template <typename T, typename WT, typename HT>
__global__ void __launch_bounds__(256)
add_rmsnorm_kernel(T* __restrict__ x, float* __restrict__ r, const HT* __restrict__ h,
                   const WT* __restrict__ w, int H, float alpha, float eps, int parts, size_t pstride, int frag_mg) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * H;
    float ss = 0.f;
    if (h != nullptr) {
        for (int j = threadIdx.x; j < H; j += 256) {
            float hs = 0.f;
            for (int p = 0; p < parts; ++p) hs += to_f32(h[p * pstride + base + j]);
            float v = r[base + j] + alpha * hs;
            r[base + j] = v;
            ss += v * v;
        }
    } else {
        for (int j = threadIdx.x; j < H; j += 256) {
            float v = r[base + j];
            ss += v * v;
        }
    }
    const float tot = block_sum<4>(ss, red);
    const float rstd = 1.0f / sqrtf(tot / (float)H + eps);
    if (frag_mg > 0) {
        // fragment order (frag.h), H a multiple of 8; the k up to the next multiple of 32 are zeros
        const int kp = (H + 31) / 32 * 32;
        for (int j = threadIdx.x; j < kp; j += 256)
            x[frag_x_chunk(blockIdx.x, j >> 3, frag_mg) * 8 + (j & 7)] = from_f32<T>(j < H ? r[base + j] * rstd * to_f32(w[j]) : 0.f);
        return;
    }
    for (int j = threadIdx.x; j < H; j += 256)
        x[base + j] = from_f32<T>(r[base + j] * rstd * to_f32(w[j]));
}

// Fast form for H = 8 * 256 * NITER' (NITER' <= NITER): each thread keeps its 8 * NITER values in
// registers between the sum of squares and the scaling, and moves 16 or 32 bytes per access.
// The order of the sum depends on H only.
template <typename T, typename WT, typename HT, int NITER>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(T* __restrict__ x, float* __restrict__ r, const HT* __restrict__ h,
                       const WT* __restrict__ w, int H, float alpha, float eps, int parts, size_t pstride, int frag_mg) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * H;
    float v[NITER][8];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * 256 + threadIdx.x) * 8;
        if (j < H) {
            const float4 r0 = *reinterpret_cast<const float4*>(r + base + j);
            const float4 r1 = *reinterpret_cast<const float4*>(r + base + j + 4);
            v[it][0] = r0.x; v[it][1] = r0.y; v[it][2] = r0.z; v[it][3] = r0.w;
            v[it][4] = r1.x; v[it][5] = r1.y; v[it][6] = r1.z; v[it][7] = r1.w;
            if (h != nullptr) {
                float hs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                // parts of a K-split product, summed in order; loaded eight at a time, so that their
                // latencies overlap (a product of many rows comes in up to 16 parts)
                constexpr int PB = 8;
                for (int p0 = 0; p0 < parts; p0 += PB) {
                    HT hv[PB][8];
#pragma unroll
                    for (int u = 0; u < PB; ++u) {
                        const int p = p0 + u < parts ? p0 + u : parts - 1;
                        const HT* hp = h + p * pstride + base + j;
                        if (sizeof(HT) == 2) {
                            *reinterpret_cast<uint4*>(hv[u]) = *reinterpret_cast<const uint4*>(hp);
                        } else {
                            *reinterpret_cast<float4*>(hv[u]) = *reinterpret_cast<const float4*>(hp);
                            *reinterpret_cast<float4*>(hv[u] + 4) = *reinterpret_cast<const float4*>(hp + 4);
                        }
                    }
#pragma unroll
                    for (int u = 0; u < PB; ++u)
                        if (p0 + u < parts) {
#pragma unroll
                            for (int e = 0; e < 8; ++e) hs[e] += to_f32(hv[u][e]);
                        }
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) v[it][e] += alpha * hs[e];
                *reinterpret_cast<float4*>(r + base + j) = make_float4(v[it][0], v[it][1], v[it][2], v[it][3]);
                *reinterpret_cast<float4*>(r + base + j + 4) = make_float4(v[it][4], v[it][5], v[it][6], v[it][7]);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += v[it][e] * v[it][e];
        }
    }
    // the weights are on their way while the sum of squares is reduced
    float wv[NITER][8];
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * 256 + threadIdx.x) * 8;
        load8<WT>(w + (j < H ? j : 0), wv[it]);
    }
    const float tot = block_sum<4>(ss, red);
    const float rstd = 1.0f / sqrtf(tot / (float)H + eps);
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * 256 + threadIdx.x) * 8;
        if (j < H) {
            T o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = from_f32<T>(v[it][e] * rstd * wv[it][e]);
            if (sizeof(T) == 2 && frag_mg > 0) {   // fragment order (frag.h): the 16-byte chunk of row blockIdx.x
                reinterpret_cast<uint4*>(x)[frag_x_chunk(blockIdx.x, j >> 3, frag_mg)] = *reinterpret_cast<uint4*>(o);
            } else if (sizeof(T) == 2) {
                *reinterpret_cast<uint4*>(x + base + j) = *reinterpret_cast<uint4*>(o);
            } else {
                *reinterpret_cast<float4*>(x + base + j) = *reinterpret_cast<float4*>(o);
                *reinterpret_cast<float4*>(x + base + j + 4) = *reinterpret_cast<float4*>(o + 4);
            }
        }
    }
    if (sizeof(T) == 2 && frag_mg > 0) {   // the k up to the next multiple of 32 are zeros
        for (int k8 = (H >> 3) + threadIdx.x; k8 < (H + 31) / 32 * 4; k8 += 256)
            reinterpret_cast<uint4*>(x)[frag_x_chunk(blockIdx.x, k8, frag_mg)] = make_uint4(0u, 0u, 0u, 0u);
    }
}

// The same for few rows of bfloat16 activations whose branch comes in many float parts (the K-split products of a
// decode step with 17 to 208 requests): a workgroup a row as above leaves most of the chip idle and walks the
// parts in several rounds of loads; here up to 16 waves take a row (as many as its width gives four columns a
// thread), and all parts' loads of a thread (up to 16) are in flight at once.  The parts are summed in ascending order; the sum of squares is
// reduced in an order that depends on H only (another one than the kernels above use: this one serves
// bfloat16 activations only, where equal bits between the kernels are not promised).
#define NORM_WIDE_THREADS 1024
#define NORM_WIDE_PARTS 16
template <typename WT, int PB>   // PB: slots for parts (8 or 16; slots beyond the parts load the last part again)
__global__ void __launch_bounds__(NORM_WIDE_THREADS)
add_rmsnorm_wide_kernel(bf16* __restrict__ x, float* __restrict__ r, const float* __restrict__ h, const WT* __restrict__ w,
                        int H, float alpha, float eps, int parts, size_t pstride, int frag_mg) {
    __shared__ float red[NORM_WIDE_THREADS / 64];
    const size_t base = (size_t)blockIdx.x * H;
    const int j = threadIdx.x * 4;
    const bool in = j < H;
    const int jc = in ? j : 0;
    float4 hv[PB];
#pragma unroll
    for (int u = 0; u < PB; ++u)
        hv[u] = *reinterpret_cast<const float4*>(h + (size_t)(u < parts ? u : parts - 1) * pstride + base + jc);
    float4 v = *reinterpret_cast<const float4*>(r + base + jc);
    float wv[4];
    if (sizeof(WT) == 2) {
        const uint2 t = *reinterpret_cast<const uint2*>(w + jc);
        wv[0] = __uint_as_float(t.x << 16); wv[1] = __uint_as_float(t.x & 0xffff0000u);
        wv[2] = __uint_as_float(t.y << 16); wv[3] = __uint_as_float(t.y & 0xffff0000u);
    } else {
        const float4 t = *reinterpret_cast<const float4*>(w + jc);
        wv[0] = t.x; wv[1] = t.y; wv[2] = t.z; wv[3] = t.w;
    }
    float4 hs = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < PB; ++u)
        if (u < parts) { hs.x += hv[u].x; hs.y += hv[u].y; hs.z += hv[u].z; hs.w += hv[u].w; }
    v.x += alpha * hs.x; v.y += alpha * hs.y; v.z += alpha * hs.z; v.w += alpha * hs.w;
    if (in) *reinterpret_cast<float4*>(r + base + j) = v;
    const float ss = in ? (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w) : 0.f;
    // over the block's waves, in wave order (their number follows from H alone)
    float tot = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = tot;
    __syncthreads();
    tot = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) tot += red[i];
    const float rstd = 1.0f / sqrtf(tot / (float)H + eps);
    bf16 o[4];
    o[0] = from_f32<bf16>(v.x * rstd * wv[0]); o[1] = from_f32<bf16>(v.y * rstd * wv[1]);
    o[2] = from_f32<bf16>(v.z * rstd * wv[2]); o[3] = from_f32<bf16>(v.w * rstd * wv[3]);
    if (frag_mg > 0) {   // fragment order (frag.h): half of the 16-byte chunk of row blockIdx.x; zeros up to the next multiple of 32 k
        const int kp = (H + 31) / 32 * 32;
        if (j < kp) {
            const uint2 val = in ? *reinterpret_cast<const uint2*>(o) : make_uint2(0u, 0u);
            *reinterpret_cast<uint2*>(reinterpret_cast<bf16*>(x) + (size_t)frag_x_chunk(blockIdx.x, j >> 3, frag_mg) * 8 + (j & 7)) = val;
        }
    } else if (in) {
        *reinterpret_cast<uint2*>(x + base + j) = *reinterpret_cast<const uint2*>(o);
    }
}

// h: the pending branch [parts][rows][H] in the activations' dtype (h_dtype == dtype) or in float
// (h_dtype == ILM_DTYPE_F32, e.g. the parts of a K-split product); null: nothing to add.
extern "C" int ilm_add_rmsnorm(void* x, void* r, const void* h, const void* w, int rows, int H,
                               float alpha, float eps, int dtype, int w_dtype, int h_dtype, int parts,
                               long pstride, int frag_mg, hipStream_t stream) {
    // frag_mg > 0: x is bfloat16 in fragment order (frag.h) with frag_mg = ceil(rows / 16) groups of rows
    ILM_REQUIRE(rows > 0 && H > 0, "add_rmsnorm: bad sizes rows=%d H=%d", rows, H);
    ILM_REQUIRE(frag_mg == 0 || (dtype == ILM_DTYPE_BF16 && H % 8 == 0 && frag_mg == (rows + 15) / 16),
                "add_rmsnorm: a result in fragment order is bfloat16 with rows of a multiple of 8 elements");
    ILM_REQUIRE(h == nullptr || (parts >= 1 && (h_dtype == dtype || h_dtype == ILM_DTYPE_F32)),
                "add_rmsnorm: the branch must have the activations' dtype or be float, in >= 1 parts");
    // H a multiple of 8 up to 8192 with 16-byte aligned rows takes the vector kernel
    const bool vec = H % 8 == 0 && H <= 8192 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)r & 15) == 0 &&
                     ((uintptr_t)h & 15) == 0 && ((uintptr_t)w & 15) == 0 && pstride % 8 == 0;
    const int niter = (H + 2047) / 2048;
    const bool hf = h != nullptr && h_dtype == ILM_DTYPE_F32;
    // few rows, many float parts, bfloat16 activations: the kernel with 16 waves a row
    if (vec && hf && dtype == ILM_DTYPE_BF16 && parts >= 4 && parts <= NORM_WIDE_PARTS && rows <= 2 * ilm_num_cus() &&
        H <= 4 * NORM_WIDE_THREADS && (H + 31) / 32 * 32 <= 4 * NORM_WIDE_THREADS) {
        const int threads = (((H + 31) / 32 * 32 / 4) + 63) / 64 * 64;   // four columns a thread, whole waves
#define NORM_WIDE(WT, PB) add_rmsnorm_wide_kernel<WT, PB><<<rows, threads, 0, stream>>>((bf16*)x, (float*)r, (const float*)h, (const WT*)w, H, alpha, eps, parts, (size_t)pstride, frag_mg)
        if (w_dtype == ILM_DTYPE_BF16) {
            if (parts <= 8) NORM_WIDE(bf16, 8); else NORM_WIDE(bf16, 16);
        } else if (w_dtype == ILM_DTYPE_F32) {
            if (parts <= 8) NORM_WIDE(float, 8); else NORM_WIDE(float, 16);
        } else
#undef NORM_WIDE
            ILM_REQUIRE(false, "add_rmsnorm: unknown dtypes %d %d", dtype, w_dtype);
        ILM_LAUNCH_CHECK("add_rmsnorm");
        return 0;
    }
#define NORM_LAUNCH(T, WT, HT)                                                                                   \
    do {                                                                                                         \
        if (vec && niter <= 1)                                                                                   \
            add_rmsnorm_vec_kernel<T, WT, HT, 1><<<rows, 256, 0, stream>>>((T*)x, (float*)r, (const HT*)h, (const WT*)w, H, alpha, eps, parts, (size_t)pstride, frag_mg); \
        else if (vec && niter <= 2)                                                                              \
            add_rmsnorm_vec_kernel<T, WT, HT, 2><<<rows, 256, 0, stream>>>((T*)x, (float*)r, (const HT*)h, (const WT*)w, H, alpha, eps, parts, (size_t)pstride, frag_mg); \
        else if (vec)                                                                                            \
            add_rmsnorm_vec_kernel<T, WT, HT, 4><<<rows, 256, 0, stream>>>((T*)x, (float*)r, (const HT*)h, (const WT*)w, H, alpha, eps, parts, (size_t)pstride, frag_mg); \
        else                                                                                                     \
            add_rmsnorm_kernel<T, WT, HT><<<rows, 256, 0, stream>>>((T*)x, (float*)r, (const HT*)h, (const WT*)w, H, alpha, eps, parts, (size_t)pstride, frag_mg); \
    } while (0)
#define NORM_CASE(T, WT)                     \
    do {                                     \
        if (hf) NORM_LAUNCH(T, WT, float);   \
        else NORM_LAUNCH(T, WT, T);          \
    } while (0)
    if (dtype == ILM_DTYPE_F32 && w_dtype == ILM_DTYPE_F32) NORM_CASE(float, float);
    else if (dtype == ILM_DTYPE_BF16 && w_dtype == ILM_DTYPE_BF16) NORM_CASE(bf16, bf16);
    else if (dtype == ILM_DTYPE_BF16 && w_dtype == ILM_DTYPE_F32) NORM_CASE(bf16, float);
    else if (dtype == ILM_DTYPE_F32 && w_dtype == ILM_DTYPE_BF16) NORM_CASE(float, bf16);
    else ILM_REQUIRE(false, "add_rmsnorm: unknown dtypes %d %d", dtype, w_dtype);
#undef NORM_CASE
#undef NORM_LAUNCH
    ILM_LAUNCH_CHECK("add_rmsnorm");
    return 0;
}

// ------------------------------------------------------------------------------------------
// Rotation of q and k in place (pairs (i, i + rd/2), tables cos/sin [max_pos, rd/2] float), and
// the write of the rotated k into the paged cache [pages, nkv, page, d] and of v into
// [pages, nkv, d, page], at slot = page_id * page + offset.  One block of 64 threads per
// (token, head slot); head slots are nh query heads, then nkv key heads, then nkv value heads, as they lie in the qkv row.
// slot < 0: nothing is written to the cache for that token.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(64)
rope_kvwrite_kernel(T* __restrict__ qkv, const int* __restrict__ pos, const float* __restrict__ cosT,
                    const float* __restrict__ sinT, T* __restrict__ kc, T* __restrict__ vc,
                    const int* __restrict__ slots, int nh, int nkv, int d, int rd, int row_stride,
                    int page) {
    const int t = blockIdx.x, hs = blockIdx.y;
    T* p = qkv + (size_t)t * row_stride + (size_t)hs * d;
    const int half = rd >> 1;
    const bool is_v = hs >= nh + nkv;
    const bool is_k = !is_v && hs >= nh;
    T* dst = nullptr;
    if (is_k && slots != nullptr) {
        const int slot = slots[t];
        if (slot >= 0) dst = kc + (((size_t)(slot / page) * nkv + (hs - nh)) * page + (slot % page)) * d;
    }
    if (is_v) {
        // values are cached transposed, [pages, nkv, d, page]: consecutive keys of one dim are contiguous
        if (slots != nullptr && slots[t] >= 0) {
            const int slot = slots[t];
            T* vdst = vc + ((size_t)(slot / page) * nkv + (hs - nh - nkv)) * d * page + (slot % page);
            for (int i = threadIdx.x; i < d; i += 64) vdst[(size_t)i * page] = p[i];
        }
        return;
    }
    const float* c = cosT + (size_t)pos[t] * half;
    const float* s = sinT + (size_t)pos[t] * half;
    for (int i = threadIdx.x; i < half; i += 64) {
        const float a = to_f32(p[i]), b = to_f32(p[i + half]);
        const T ra = from_f32<T>(a * c[i] - b * s[i]);
        const T rb = from_f32<T>(b * c[i] + a * s[i]);
        p[i] = ra;
        p[i + half] = rb;
        if (dst != nullptr) {
            dst[i] = ra;
            dst[i + half] = rb;
        }
    }
    if (dst != nullptr)
        for (int i = rd + threadIdx.x; i < d; i += 64) dst[i] = p[i];
}

// Vector form: one block a token, every thread 8 consecutive dims of a pair (16-byte accesses).
// Needs rd a multiple of 16 (half the rotary dims in steps of 8) and d a multiple of 8.
template <typename T>
__device__ __forceinline__ void store8(T* p, const T* t) {
    if (sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(t);
    } else {
        *reinterpret_cast<float4*>(p) = *reinterpret_cast<const float4*>(t);
        *reinterpret_cast<float4*>(p + 4) = *reinterpret_cast<const float4*>(t + 4);
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
rope_kvwrite_vec_kernel(T* __restrict__ qkv, const int* __restrict__ pos, const float* __restrict__ cosT,
                        const float* __restrict__ sinT, T* __restrict__ kc, T* __restrict__ vc,
                        const int* __restrict__ slots, int nh, int nkv, int d, int rd, int row_stride, int page) {
    const int t = blockIdx.x;
    const int half = rd >> 1;
    const int hp = half >> 3;              // 8-wide pieces of a rotated pair per head
    const int tail = (d - rd) >> 3;        // 8-wide pieces of a head that are not rotated
    const int per_qk = hp + tail;          // work items of a q or k head
    const int per_v = d >> 3;
    const int slot = slots != nullptr ? slots[t] : -1;
    const int n_items = (nh + nkv) * per_qk + nkv * per_v;
    const float* c = cosT + (size_t)pos[t] * half;
    const float* s = sinT + (size_t)pos[t] * half;
    T* row = qkv + (size_t)t * row_stride;
    for (int it = threadIdx.x; it < n_items; it += 256) {
        if (it < (nh + nkv) * per_qk) {
            const int hs = it / per_qk, piece = it % per_qk;
            T* p = row + (size_t)hs * d;
            T* dst = nullptr;
            if (hs >= nh && slot >= 0) dst = kc + (((size_t)(slot / page) * nkv + (hs - nh)) * page + (slot % page)) * d;
            if (piece < hp) {
                const int i = piece * 8;
                float a[8], b[8], cc[8], ss[8];
                load8(p + i, a);
                load8(p + i + half, b);
                load8(c + i, cc);
                load8(s + i, ss);
                T ra[8], rb[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    ra[e] = from_f32<T>(a[e] * cc[e] - b[e] * ss[e]);
                    rb[e] = from_f32<T>(b[e] * cc[e] + a[e] * ss[e]);
                }
                store8(p + i, ra);
                store8(p + i + half, rb);
                if (dst != nullptr) {
                    store8(dst + i, ra);
                    store8(dst + i + half, rb);
                }
            } else if (dst != nullptr) {
                const int i = rd + (piece - hp) * 8;
                T v8[8];
                store8(v8, p + i);
                store8(dst + i, v8);
            }
        } else if (slot >= 0) {
            const int j = it - (nh + nkv) * per_qk;
            const int kvh = j / per_v, i = (j % per_v) * 8;
            T v8[8];
            store8(v8, row + (size_t)(nh + nkv + kvh) * d + i);
            T* vdst = vc + ((size_t)(slot / page) * nkv + kvh) * d * page + (slot % page);
#pragma unroll
            for (int e = 0; e < 8; ++e) vdst[(size_t)(i + e) * page] = v8[e];
        }
    }
}

extern "C" int ilm_rope_kvwrite(void* qkv, const void* pos, const void* cosT, const void* sinT,
                                void* kc, void* vc, const void* slots, int T_, int nh, int nkv,
                                int d, int rd, int row_stride, int page, int dtype,
                                hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv >= 0 && d > 0, "rope_kvwrite: bad sizes");
    ILM_REQUIRE(rd >= 0 && rd <= d && rd % 2 == 0, "rope_kvwrite: rotary dim %d does not fit head dim %d", rd, d);
    ILM_REQUIRE(row_stride >= (nh + 2 * nkv) * d, "rope_kvwrite: row stride %d too small", row_stride);
    ILM_REQUIRE(slots == nullptr || page > 0, "rope_kvwrite: page size %d", page);
    const bool vec = rd % 16 == 0 && d % 8 == 0 && row_stride % 8 == 0 && ((uintptr_t)qkv & 31) == 0 &&
                     ((uintptr_t)kc & 31) == 0 && ((uintptr_t)cosT & 31) == 0 && ((uintptr_t)sinT & 31) == 0;
    if (vec && dtype == ILM_DTYPE_F32) {
        rope_kvwrite_vec_kernel<float><<<T_, 256, 0, stream>>>((float*)qkv, (const int*)pos, (const float*)cosT,
                                                              (const float*)sinT, (float*)kc, (float*)vc,
                                                              (const int*)slots, nh, nkv, d, rd, row_stride, page);
        ILM_LAUNCH_CHECK("rope_kvwrite");
        return 0;
    }
    if (vec && dtype == ILM_DTYPE_BF16) {
        rope_kvwrite_vec_kernel<bf16><<<T_, 256, 0, stream>>>((bf16*)qkv, (const int*)pos, (const float*)cosT,
                                                             (const float*)sinT, (bf16*)kc, (bf16*)vc,
                                                             (const int*)slots, nh, nkv, d, rd, row_stride, page);
        ILM_LAUNCH_CHECK("rope_kvwrite");
        return 0;
    }
    dim3 grid(T_, nh + 2 * nkv);
    if (dtype == ILM_DTYPE_F32)
        rope_kvwrite_kernel<float><<<grid, 64, 0, stream>>>((float*)qkv, (const int*)pos, (const float*)cosT,
                                                           (const float*)sinT, (float*)kc, (float*)vc,
                                                           (const int*)slots, nh, nkv, d, rd, row_stride, page);
    else if (dtype == ILM_DTYPE_BF16)
        rope_kvwrite_kernel<bf16><<<grid, 64, 0, stream>>>((bf16*)qkv, (const int*)pos, (const float*)cosT,
                                                          (const float*)sinT, (bf16*)kc, (bf16*)vc,
                                                          (const int*)slots, nh, nkv, d, rd, row_stride, page);
    else
        ILM_REQUIRE(false, "rope_kvwrite: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("rope_kvwrite");
    return 0;
}

// ------------------------------------------------------------------------------------------
// act[t, i] = silu(gu[t, i]) * gu[t, I + i]   (gate is the first half of the fused projection)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(T* __restrict__ out, const T* __restrict__ gu, int I, int gu_stride) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= I) return;
    const float g = to_f32(gu[(size_t)t * gu_stride + i]);
    const float u = to_f32(gu[(size_t)t * gu_stride + I + i]);
    out[(size_t)t * I + i] = from_f32<T>(g / (1.0f + expf(-g)) * u);
}

// 8 elements a thread, 16-byte (bf16) or 32-byte (float) accesses; needs I and the row stride to be
// multiples of 8 and 16-byte aligned rows
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_vec_kernel(T* __restrict__ out, const T* __restrict__ gu, int I, int gu_stride) {
    const int t = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= I) return;
    T g[8], u[8], o[8];
    const T* gp = gu + (size_t)t * gu_stride + i;
    if (sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(g) = *reinterpret_cast<const uint4*>(gp);
        *reinterpret_cast<uint4*>(u) = *reinterpret_cast<const uint4*>(gp + I);
    } else {
        *reinterpret_cast<float4*>(g) = *reinterpret_cast<const float4*>(gp);
        *reinterpret_cast<float4*>(g + 4) = *reinterpret_cast<const float4*>(gp + 4);
        *reinterpret_cast<float4*>(u) = *reinterpret_cast<const float4*>(gp + I);
        *reinterpret_cast<float4*>(u + 4) = *reinterpret_cast<const float4*>(gp + I + 4);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float gv = to_f32(g[e]);
        o[e] = from_f32<T>(gv / (1.0f + expf(-gv)) * to_f32(u[e]));
    }
    T* op = out + (size_t)t * I + i;
    if (sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(op) = *reinterpret_cast<uint4*>(o);
    } else {
        *reinterpret_cast<float4*>(op) = *reinterpret_cast<float4*>(o);
        *reinterpret_cast<float4*>(op + 4) = *reinterpret_cast<float4*>(o + 4);
    }
}

extern "C" int ilm_swiglu(void* out, const void* gu, int T_, int I, int gu_stride, int dtype,
                          hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && I > 0 && gu_stride >= 2 * I, "swiglu: bad sizes T=%d I=%d stride=%d", T_, I, gu_stride);
    ILM_REQUIRE(T_ <= 65535, "swiglu: at most 65535 rows a call, got %d", T_);
    const bool vec = I % 8 == 0 && gu_stride % 8 == 0 && ((uintptr_t)out & 31) == 0 && ((uintptr_t)gu & 31) == 0;
    dim3 grid((I + 255) / 256, T_);
    dim3 vgrid((I / 8 + 255) / 256, T_);
    if (dtype == ILM_DTYPE_F32 && vec)
        swiglu_vec_kernel<float><<<vgrid, 256, 0, stream>>>((float*)out, (const float*)gu, I, gu_stride);
    else if (dtype == ILM_DTYPE_BF16 && vec)
        swiglu_vec_kernel<bf16><<<vgrid, 256, 0, stream>>>((bf16*)out, (const bf16*)gu, I, gu_stride);
    else if (dtype == ILM_DTYPE_F32)
        swiglu_kernel<float><<<grid, 256, 0, stream>>>((float*)out, (const float*)gu, I, gu_stride);
    else if (dtype == ILM_DTYPE_BF16)
        swiglu_kernel<bf16><<<grid, 256, 0, stream>>>((bf16*)out, (const bf16*)gu, I, gu_stride);
    else
        ILM_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("swiglu");
    return 0;
}

// ------------------------------------------------------------------------------------------
// out[i, :] = in[idx[i], :]
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void gather_rows_kernel(T* __restrict__ out, const T* __restrict__ in,
                                   const int* __restrict__ idx, int H) {
    const T* src = in + (size_t)idx[blockIdx.x] * H;
    T* dst = out + (size_t)blockIdx.x * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = src[j];
}

extern "C" int ilm_gather_rows(void* out, const void* in, const void* idx, int n, int H, int dtype,
                               hipStream_t stream) {
    ILM_REQUIRE(n > 0 && H > 0, "gather_rows: bad sizes n=%d H=%d", n, H);
    if (dtype == ILM_DTYPE_F32)
        gather_rows_kernel<float><<<n, 256, 0, stream>>>((float*)out, (const float*)in, (const int*)idx, H);
    else if (dtype == ILM_DTYPE_BF16)
        gather_rows_kernel<bf16><<<n, 256, 0, stream>>>((bf16*)out, (const bf16*)in, (const int*)idx, H);
    else
        ILM_REQUIRE(false, "gather_rows: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("gather_rows");
    return 0;
}

// ------------------------------------------------------------------------------------------
// x[i, :n] *= alpha over rows of float (the output head's scale after a library product)
// ------------------------------------------------------------------------------------------
__global__ void scale_rows_kernel(float* __restrict__ x, int cols, int stride, float alpha) {
    float* row = x + (size_t)blockIdx.y * stride;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < cols) row[j] *= alpha;
}

extern "C" int ilm_scale_rows(void* x, int rows, int cols, int stride, float alpha, hipStream_t stream) {
    ILM_REQUIRE(rows > 0 && rows <= 65535 && cols > 0 && stride >= cols, "scale_rows: bad sizes rows=%d cols=%d stride=%d",
                rows, cols, stride);
    scale_rows_kernel<<<dim3((cols + 255) / 256, rows), 256, 0, stream>>>((float*)x, cols, stride, alpha);
    ILM_LAUNCH_CHECK("scale_rows");
    return 0;
}
