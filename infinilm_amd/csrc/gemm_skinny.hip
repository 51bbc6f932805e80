// C[M,N] = alpha * (X[M,K] W[N,K]^T + bias) for few rows of X (M <= 64), bfloat16 in, float
// accumulation: the decode-side projection, bound by reading W once from HBM.
//
// One workgroup of 8 waves owns 16 rows of W (16 outputs for every token).  The waves split K into
// 8 contiguous slices; each streams its slice of the 16 rows straight from global memory into MFMA
// operands (v_mfma_f32_16x16x32_bf16: W rows on the A side, tokens on the B side, 16 tokens per
// accumulator, up to 4 accumulators), with every load of a chunk issued before the chunk's first
// MFMA.  The 8 partial tiles are summed through LDS in wave order, so the result is deterministic.
// The X fragments come from L2 (X is at most 64 x K).
// K must be a multiple of 8 (16-byte loads); rows of X and W must be 16-byte aligned.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define SK_WAVES 8
#define SK_UNROLL 4

template <int MG, typename TC>
__global__ void __launch_bounds__(SK_WAVES * 64)
gemm_skinny_kernel(TC* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W,
                   const bf16* __restrict__ bias, int M, int N, int K, int lda, int ldw, int ldc,
                   float alpha) {
    __shared__ float part[SK_WAVES][MG][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int steps_total = (K + 31) >> 5;
    const int per = (steps_total + SK_WAVES - 1) / SK_WAVES;
    const int s0 = wave * per;
    const int s1 = (s0 + per < steps_total) ? s0 + per : steps_total;

    const int wrow = (n0 + r < N) ? n0 + r : N - 1;
    const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)wrow * ldw);
    const uint4* xp[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        const int m = (g * 16 + r < M) ? g * 16 + r : M - 1;
        xp[g] = reinterpret_cast<const uint4*>(X + (size_t)m * lda);
    }
    f32x4 acc[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};

    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    for (int s = s0; s < s1; s += SK_UNROLL) {
        uint4 a[SK_UNROLL];
        uint4 b[SK_UNROLL][MG];
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u) {
            const int k8 = (s + u) * 4 + q;  // index of this lane's group of 8 elements
            const bool ok = (s + u < s1) && (k8 * 8 + 8 <= K);
            a[u] = ok ? wp[k8] : zero;
#pragma unroll
            for (int g = 0; g < MG; ++g) b[u][g] = ok ? xp[g][k8] : zero;
        }
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
            for (int g = 0; g < MG; ++g)
                acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[u]),
                                                                 __builtin_bit_cast(bf16x8, b[u][g]), acc[g], 0, 0, 0);
    }
#pragma unroll
    for (int g = 0; g < MG; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) part[wave][g][lane][e] = acc[g][e];
    __syncthreads();
    // acc[g][e] of lane (r, q) is output row n0 + q*4 + e for token g*16 + r
    for (int idx = threadIdx.x; idx < MG * 64 * 4; idx += SK_WAVES * 64) {
        const int e = idx & 3, l = (idx >> 2) & 63, g = idx >> 8;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) v += part[w][g][l][e];
        const int n = n0 + (l >> 4) * 4 + e;
        const int m = g * 16 + (l & 15);
        if (n < N && m < M) {
            if (bias != nullptr) v += to_f32(bias[n]);
            C[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
        }
    }
}

extern "C" int ilm_gemm_skinny(void* C, const void* X, const void* W, const void* bias, int M, int N,
                               int K, int lda, int ldw, int ldc, float alpha, int out_dtype,
                               hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: needs 1 <= M <= 64, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_skinny: K=%d lda=%d ldw=%d must be multiples of 8",
                K, lda, ldw);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_skinny: operands must be 16-byte aligned");
    ILM_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_skinny: strides too small");
    const int grid = (N + 15) / 16;
    const int mg = (M + 15) / 16;
#define SK_CASE(MG, TC)                                                                                   \
    gemm_skinny_kernel<MG, TC><<<grid, SK_WAVES * 64, 0, stream>>>((TC*)C, (const bf16*)X, (const bf16*)W, \
                                                                   (const bf16*)bias, M, N, K, lda, ldw, ldc, alpha)
#define SK_DISPATCH(TC)             \
    switch (mg) {                   \
        case 1: SK_CASE(1, TC); break; \
        case 2: SK_CASE(2, TC); break; \
        case 3: SK_CASE(3, TC); break; \
        default: SK_CASE(4, TC); break; \
    }
    if (out_dtype == ILM_DTYPE_BF16) { SK_DISPATCH(bf16) }
    else if (out_dtype == ILM_DTYPE_F32) { SK_DISPATCH(float) }
    else ILM_REQUIRE(false, "gemm_skinny: unknown output dtype %d", out_dtype);
#undef SK_DISPATCH
#undef SK_CASE
    ILM_LAUNCH_CHECK("gemm_skinny");
    return 0;
}
