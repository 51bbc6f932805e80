// The projection that ends a branch (few rows of X, bfloat16) with the residual sum and the first
// half of the following RMS norm in its epilogue: one kernel less between the branch and the part
// after the norm.
//
//   r[m, n]  <-  r[m, n] + alpha * (X W^T + bias)[m, n]        the float residual stream, in place
//   xw[m, n]  =  bfloat16(r[m, n] * w[n])                       w: the weight of the norm that follows
//   ss[tile, m] = sum over the tile's 16 outputs of r[m, n]^2   partial sums of squares of the rows
//
// The norm's division by the root mean square is one number a row; the product that consumes xw
// applies it to its sums (rstd * (V xw) = V (rstd xw)) after adding up the partial sums of squares
// in tile order (gemm_skinny.hip: the gate/up kernels).  The product itself is the resident
// few-rows one (X fragments in registers, W streamed once on v_mfma_f32_16x16x32_bf16, K split over
// the waves and reduced through LDS in wave order), in which every output has one owner: the sum
// into the residual needs no atomics and keeps its order.  M <= 16 with K <= 8192, or M <= 32
// with K <= 4096.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define GT_SS_ROWS 32   // rows of a tile's record of partial sums (the most rows the kernel takes)

__device__ __forceinline__ f32x4 gt_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <int WAVES, int KSTEPS, int MG, typename NWT>
__global__ void __launch_bounds__(WAVES * 64)
gemm_tail_kernel(float* __restrict__ R, bf16* __restrict__ XW, float* __restrict__ SS, const bf16* __restrict__ X,
                 const bf16* __restrict__ W, const bf16* __restrict__ bias, const NWT* __restrict__ nw, int M, int N, int K,
                 int lda, int ldw, int ldr, int ldxw, float alpha, int ntiles, int ks) {
    // ks <= KSTEPS: k-steps a wave really takes (K spread evenly over the waves); its other slots load
    // its first address again (a cache hit, no branch around the loads) and multiply by zeros
    static_assert(WAVES * 64 >= 256 * MG, "one reducing thread an output");
    __shared__ float part[2][MG][WAVES][64][4];
    __shared__ float ssred[2][MG][4][16];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int s0 = wave * ks;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (K >> 3) - 1;
    int k8c[KSTEPS];
    bool kok[KSTEPS];
#pragma unroll
    for (int u = 0; u < KSTEPS; ++u) {
        const int k8 = (s0 + u) * 4 + q;
        kok[u] = u < ks && k8 <= k8_last;
        k8c[u] = kok[u] ? k8 : (u == 0 ? k8_last : k8c[0]);
    }
    // the first W tile is on its way before the X fragments
    uint4 a[KSTEPS];
    int tile = blockIdx.x;
    if (tile < ntiles) {
        const int row = (tile * 16 + r < N) ? tile * 16 + r : N - 1;
        const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)row * ldw);
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
    }
    uint4 xf[MG][KSTEPS];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        const int row = g * 16 + r;
        const uint4* xp = reinterpret_cast<const uint4*>(X + (size_t)(row < M ? row : 0) * lda);
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u) {
            const uint4 v = xp[k8c[u]];
            // zero fragments beyond K or beyond M make the clamped W loads harmless
            xf[g][u] = (kok[u] && row < M) ? v : zero;
        }
    }
    // the epilogue thread's output: row m, output (j, e) of the tile
    const bool reducer = threadIdx.x < 256 * MG;
    const int et = reducer ? threadIdx.x : 0;
    const int eg = et >> 8, t8 = et & 255, e = t8 & 3, l = t8 >> 2;
    const int m16 = l & 15, j = l >> 4, m = eg * 16 + m16;
    int buf = 0;
    for (; tile < ntiles; tile += gridDim.x) {
        // the epilogue's own operands are on their way while the tile is multiplied
        const int n = tile * 16 + j * 4 + e;
        const bool writer = reducer && n < N && m < M;
        float* rp = R + (size_t)(writer ? m : 0) * ldr + (writer ? n : 0);
        const float r_old = *rp;
        const float w_n = to_f32(nw[writer ? n : 0]);
        const float b_n = (bias != nullptr) ? to_f32(bias[writer ? n : 0]) : 0.f;
        f32x4 acc[MG];
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u)
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[g] = gt_mfma(a[u], xf[g][u], acc[g]);
        // the next tile's rows are on their way while this one is reduced
        const int next = tile + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        if (next < ntiles) {
            const int row = (next * 16 + r < N) ? next * 16 + r : N - 1;
            const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)row * ldw);
#pragma unroll
            for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[buf][g][wave][lane][0]) = acc[g];
        __syncthreads();
        float sq = 0.f;
        if (reducer) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) v += part[buf][eg][w][l][e];
            if (writer) {
                const float rn = fmaf(alpha, v + b_n, r_old);
                *rp = rn;
                XW[(size_t)m * ldxw + n] = from_f32<bf16>(rn * w_n);
                sq = rn * rn;
            }
            // over the four outputs of a lane group (e), then over the four groups (j: one wave each)
            sq += __shfl_xor(sq, 1, 64);
            sq += __shfl_xor(sq, 2, 64);
            if (e == 0) ssred[buf][eg][j][m16] = sq;
        }
        __syncthreads();
        if (reducer && j == 0 && e == 0)
            SS[(size_t)tile * GT_SS_ROWS + m] = (ssred[buf][eg][0][m16] + ssred[buf][eg][1][m16]) +
                                                (ssred[buf][eg][2][m16] + ssred[buf][eg][3][m16]);
        buf ^= 1;  // the other buffers are free: their readers passed a barrier above one tile ago
    }
}

extern "C" int ilm_gemm_tail_ss_rows() { return GT_SS_ROWS; }

// R [M, ldr] float in/out; XW [M, ldxw] bfloat16 out; SS [ceil(N / 16), ilm_gemm_tail_ss_rows()] float out (rows
// beyond M are not written); norm_w [N] of dtype nw_dtype.
extern "C" int ilm_gemm_tail(void* R, int ldr, void* XW, int ldxw, void* SS, const void* X, int lda, const void* W, int ldw,
                             const void* bias, const void* norm_w, int nw_dtype, float alpha, int M, int N, int K,
                             hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 32 && N > 0 && K > 0, "gemm_tail: needs 1 <= M <= 32, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldr >= N && ldxw >= N,
                "gemm_tail: K=%d lda=%d ldw=%d ldr=%d ldxw=%d", K, lda, ldw, ldr, ldxw);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_tail: operands must be 16-byte aligned");
    ILM_REQUIRE(nw_dtype == ILM_DTYPE_F32 || nw_dtype == ILM_DTYPE_BF16, "gemm_tail: unknown norm weight dtype %d", nw_dtype);
    ILM_REQUIRE(R != nullptr && XW != nullptr && SS != nullptr && norm_w != nullptr, "gemm_tail: null operand");
    const int ksteps = (K + 31) / 32;
    ILM_REQUIRE((M <= 16 && ksteps <= 16 * 16) || ksteps <= 8 * 16, "gemm_tail: K=%d is beyond %d", K, M <= 16 ? 8192 : 4096);
    const int ntiles = (N + 15) / 16;
#define GT_LAUNCH(WV, KS, MGR, PER_CU, NWT)                                                                       \
    {                                                                                                             \
        const int grid = ntiles < ilm_num_cus() * PER_CU ? ntiles : ilm_num_cus() * PER_CU;                         \
        gemm_tail_kernel<WV, KS, MGR, NWT><<<grid, WV * 64, 0, stream>>>(                                         \
            (float*)R, (bf16*)XW, (float*)SS, (const bf16*)X, (const bf16*)W, (const bf16*)bias, (const NWT*)norm_w, \
            M, N, K, lda, ldw, ldr, ldxw, alpha, ntiles, (ksteps + WV - 1) / WV);                                 \
    }
#define GT_CASE(WV, KS, MGR, PER_CU)                                           \
    {                                                                          \
        if (nw_dtype == ILM_DTYPE_F32) GT_LAUNCH(WV, KS, MGR, PER_CU, float)   \
        else GT_LAUNCH(WV, KS, MGR, PER_CU, bf16)                              \
    }
    if (M > 16) {
        if (ksteps <= 8 * 4) GT_CASE(8, 4, 2, 2)
        else if (ksteps <= 8 * 8) GT_CASE(8, 8, 2, 2)
        else if (ksteps <= 8 * 12) GT_CASE(8, 12, 2, 1)
        else GT_CASE(8, 16, 2, 1)
    }
    else if (ksteps <= 8 * 4) GT_CASE(8, 4, 1, 2)
    else if (ksteps <= 8 * 8) GT_CASE(8, 8, 1, 2)
    else if (ksteps <= 8 * 12) GT_CASE(8, 12, 1, 2)
    else if (ksteps <= 8 * 16) GT_CASE(8, 16, 1, 2)
    else if (ksteps <= 16 * 12) GT_CASE(16, 12, 1, 1)
    else GT_CASE(16, 16, 1, 1)
#undef GT_LAUNCH
#undef GT_CASE
    ILM_LAUNCH_CHECK("gemm_tail");
    return 0;
}
