// C[M,N] = alpha * (A[M,K] W[N,K]^T + bias[N]) with float multiply-adds in ascending k: the 32-bit
// path of every projection, and the fallback for bf16 shapes the MFMA kernels refuse.  An output
// element's sum is formed in the same order whatever M and N are, so logits do not depend on
// how tokens were batched.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_nt_basic_kernel(TC* __restrict__ C, const TA* __restrict__ A, const TW* __restrict__ W,
                     const TW* __restrict__ bias, int M, int N, int K, int lda, int ldw, int ldc,
                     float alpha) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + i * 256;
            const int row = idx >> 4, kk = idx & 15;
            const int k = k0 + kk;
            float a = 0.f, w = 0.f;
            if (k < K) {
                if (m0 + row < M) a = to_f32(A[(size_t)(m0 + row) * lda + k]);
                if (n0 + row < N) w = to_f32(W[(size_t)(n0 + row) * ldw + k]);
            }
            As[kk][row] = a;
            Ws[kk][row] = w;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias != nullptr) v += to_f32(bias[n]);
            C[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
        }
    }
}

extern "C" int ilm_gemm_basic(void* C, const void* A, const void* W, const void* bias, int M, int N,
                              int K, int lda, int ldw, int ldc, float alpha, int in_dtype,
                              int out_dtype, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: strides lda=%d ldw=%d ldc=%d too small for K=%d N=%d",
                lda, ldw, ldc, K, N);
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    ILM_REQUIRE(grid.y <= 65535, "gemm: M=%d too large for one call", M);
#define GEMM_CASE(TA, TW, TC)                                                                     \
    gemm_nt_basic_kernel<TA, TW, TC><<<grid, 256, 0, stream>>>((TC*)C, (const TA*)A, (const TW*)W, \
                                                               (const TW*)bias, M, N, K, lda, ldw, ldc, alpha)
    if (in_dtype == ILM_DTYPE_F32 && out_dtype == ILM_DTYPE_F32) GEMM_CASE(float, float, float);
    else if (in_dtype == ILM_DTYPE_BF16 && out_dtype == ILM_DTYPE_BF16) GEMM_CASE(bf16, bf16, bf16);
    else if (in_dtype == ILM_DTYPE_BF16 && out_dtype == ILM_DTYPE_F32) GEMM_CASE(bf16, bf16, float);
    else ILM_REQUIRE(false, "gemm: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
#undef GEMM_CASE
    ILM_LAUNCH_CHECK("gemm_basic");
    return 0;
}
