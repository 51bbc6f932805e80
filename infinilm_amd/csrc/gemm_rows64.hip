// C[y][M][N] (float32 parts) = X[M, K-range y] W[N, K-range y]^T for 33 to 64 rows of X, bfloat16: the
// o and down projections of a decode step with many requests, whose results go into the residual
// sum (the next add+RMSNorm sums the parts).
//
// With so many rows the X fragments of a whole K no longer fit the registers, so K is cut into
// ranges of R6_SPAN over blockIdx.y: a wave keeps the X fragments of its R6_KS k-steps for all four
// groups of 16 rows (64 registers) and multiplies R6_T tiles of 16 W rows at once (64 registers of
// W fragments in flight, as many bytes a wave as the few-rows kernels keep in flight with one tile
// of a long K).  X is read once a workgroup; a W fragment read once serves four matrix instructions.
// The eight waves' partial tiles are summed through LDS in wave order (deterministic).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define R6_WAVES 8
#define R6_KS 4
#define R6_T 4
#define R6_MG 4
#define R6_SPAN (R6_WAVES * R6_KS * 32)   // 1024

__device__ __forceinline__ f32x4 r6_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// FRAGW: W is given in fragment order (frag.h), tiles of 16 consecutive rows: a wave's W fragment is 1 KB of
// consecutive bytes (a compute unit takes those in several times faster than fragments gathered from rows).
template <bool FRAGW>
__global__ void __launch_bounds__(R6_WAVES * 64)
gemm_rows64_kernel(float* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W, int M, int N, int K,
                   int lda, int ldw, int ldc, size_t c_part_stride, int n_groups) {
    __shared__ float part[2][R6_MG][R6_WAVES][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int kslice = blockIdx.y;
    const int k_lo = kslice * R6_SPAN;
    const int k_hi = (k_lo + R6_SPAN < K) ? k_lo + R6_SPAN : K;
    const int k8_first = k_lo >> 3, k8_last = (k_hi >> 3) - 1;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    int k8c[R6_KS];
    bool kok[R6_KS];
#pragma unroll
    for (int u = 0; u < R6_KS; ++u) {
        const int k8 = k8_first + (wave * R6_KS + u) * 4 + q;
        kok[u] = k8 <= k8_last;
        k8c[u] = kok[u] ? k8 : k8_last;
    }
    const int ntiles = (N + 15) / 16;
    const int ksteps = (K + 31) >> 5;
    int wk[R6_KS];   // where a step's W fragment lies from the tile's (FRAGW) or the row's start, in 16-byte units
#pragma unroll
    for (int u = 0; u < R6_KS; ++u) wk[u] = FRAGW ? (k8c[u] >> 2) * 64 : k8c[u];
    // this lane's W row of tile t of a group (clamped: rows beyond N are never stored)
    auto w_row = [&](int group, int t) -> const uint4* {
        if (FRAGW) {
            int tile = group * R6_T + t;
            tile = tile < ntiles ? tile : ntiles - 1;
            return reinterpret_cast<const uint4*>(W) + (size_t)tile * ksteps * 64 + lane;
        }
        int n = (group * R6_T + t) * 16 + r;
        n = n < N ? n : N - 1;
        return reinterpret_cast<const uint4*>(W + (size_t)n * ldw);
    };
    uint4 a[R6_T][R6_KS];
    int group = blockIdx.x;
    if (group < n_groups) {
#pragma unroll
        for (int t = 0; t < R6_T; ++t) {
            const uint4* wp = w_row(group, t);
#pragma unroll
            for (int u = 0; u < R6_KS; ++u) a[t][u] = wp[wk[u]];
        }
    }
    uint4 xf[R6_MG][R6_KS];
#pragma unroll
    for (int g = 0; g < R6_MG; ++g) {
        const int row = g * 16 + r;
        const uint4* xp = reinterpret_cast<const uint4*>(X + (size_t)(row < M ? row : 0) * lda);
#pragma unroll
        for (int u = 0; u < R6_KS; ++u) {
            const uint4 v = xp[k8c[u]];
            xf[g][u] = (kok[u] && row < M) ? v : zero;   // zero fragments make the clamped W loads harmless
        }
    }
    float* Cp = C + (size_t)kslice * c_part_stride;
    int buf = 0;
    for (; group < n_groups; group += gridDim.x) {
        f32x4 acc[R6_T][R6_MG];
#pragma unroll
        for (int t = 0; t < R6_T; ++t)
#pragma unroll
            for (int g = 0; g < R6_MG; ++g) acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < R6_KS; ++u)
#pragma unroll
            for (int t = 0; t < R6_T; ++t)
#pragma unroll
                for (int g = 0; g < R6_MG; ++g) acc[t][g] = r6_mfma(a[t][u], xf[g][u], acc[t][g]);
        // the next group's rows are on their way while this one is reduced
        const int next = group + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        if (next < n_groups) {
#pragma unroll
            for (int t = 0; t < R6_T; ++t) {
                const uint4* wp = w_row(next, t);
#pragma unroll
                for (int u = 0; u < R6_KS; ++u) a[t][u] = wp[wk[u]];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < R6_T; ++t) {
#pragma unroll
            for (int g = 0; g < R6_MG; ++g) *reinterpret_cast<f32x4*>(&part[buf][g][wave][lane][0]) = acc[t][g];
            __syncthreads();
            const int tile = group * R6_T + t;
#pragma unroll
            for (int half = 0; half < 2; ++half) {   // 1024 outputs a tile, two a thread
                const int idx = threadIdx.x + half * 512;
                const int g = idx >> 8, e = idx & 3, l = (idx & 255) >> 2;
                float v = 0.f;
#pragma unroll
                for (int w = 0; w < R6_WAVES; ++w) v += part[buf][g][w][l][e];
                const int n = tile * 16 + (l >> 4) * 4 + e;
                const int m = g * 16 + (l & 15);
                if (tile < ntiles && n < N && m < M) Cp[(size_t)m * ldc + n] = v;
            }
            buf ^= 1;  // the other buffer is free: its readers passed the barrier above one tile ago
        }
    }
}

extern "C" int ilm_gemm_rows64_span() { return R6_SPAN; }

// C: float [kb][M][ldc] with c_part_stride elements between the parts, kb = ceil(K / ilm_gemm_rows64_span()).
// frag_w != 0: W is the weight in fragment order, tiles of 16 consecutive rows (ldw is not used).
extern "C" int ilm_gemm_rows64(void* C, int ldc, long c_part_stride, int kb, const void* W, int ldw, int M, int N, int K,
                               const void* X, int lda, int frag_w, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_rows64: needs 1 <= M <= 64, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && (frag_w || (ldw % 8 == 0 && ldw >= K)) && lda >= K && ldc >= N,
                "gemm_rows64: K=%d lda=%d ldw=%d ldc=%d", K, lda, ldw, ldc);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_rows64: operands must be 16-byte aligned");
    ILM_REQUIRE(kb == (K + R6_SPAN - 1) / R6_SPAN && kb <= 65535, "gemm_rows64: K=%d needs %d parts, got %d", K,
                (K + R6_SPAN - 1) / R6_SPAN, kb);
    const int ntiles = (N + 15) / 16;
    const int n_groups = (ntiles + R6_T - 1) / R6_T;
    int gx = ilm_num_cus() / kb;
    if (gx < 1) gx = 1;
    if (gx > n_groups) gx = n_groups;
    dim3 grid(gx, kb);
    if (frag_w)
        gemm_rows64_kernel<true><<<grid, R6_WAVES * 64, 0, stream>>>((float*)C, (const bf16*)X, (const bf16*)W, M, N, K, lda, ldw,
                                                                     ldc, (size_t)c_part_stride, n_groups);
    else
        gemm_rows64_kernel<false><<<grid, R6_WAVES * 64, 0, stream>>>((float*)C, (const bf16*)X, (const bf16*)W, M, N, K, lda, ldw,
                                                                      ldc, (size_t)c_part_stride, n_groups);
    ILM_LAUNCH_CHECK("gemm_rows64");
    return 0;
}
