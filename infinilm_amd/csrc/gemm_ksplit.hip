// The decode-side projection (at most 32 rows of X, bfloat16) for long K: blockIdx.y takes a
// contiguous K range of GF_KSPAN and writes a float partial result C[y][M][N]; the consumer (the next
// add+RMSNorm) sums the parts in order.  Within a range the kernel is the resident few-rows
// product: W streamed once on v_mfma_f32_16x16x32_bf16, the X fragments in registers, the next W
// row tile prefetched while the previous one is reduced.  This gives the long-K product
// (down_proj) the shape of the short-K ones instead of 64 k-steps a wave.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

#define GF_KSPAN 4096   // K a workgroup covers: waves x k-steps x 32

__device__ __forceinline__ f32x4 gf_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
// 16 waves x 8 k-steps keep a wave under 128 registers (4 waves a SIMD, one workgroup a CU); with two
// groups of 16 rows of X (MG = 2) it is 8 waves x 16 k-steps under 256 registers.
// ACT: X holds rows [gate | up] of 2K elements and the fragment is made on the fly,
// x = silu(gate) * up (the SwiGLU between the two projections of a feed-forward), instead of being
// read: one kernel and one trip through memory less a layer.
template <int GF_WAVES, int GF_KSTEPS, int MG, bool ACT, typename TC>
__global__ void __launch_bounds__(GF_WAVES * 64)
gemm_ksplit_kernel(TC* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W,
                   const bf16* __restrict__ bias, int M, int N, int K, int lda, int ldw, int ldc, float alpha,
                   int ntiles, size_t c_part_stride, int kspan, int ks) {
    // kspan <= GF_KSPAN: K a part really covers (K spread evenly over the parts, a multiple of 32);
    // ks <= GF_KSTEPS: k-steps a wave really takes (the part spread evenly over the waves); its other
    // slots load its first address again (a cache hit, no branch around the loads) and multiply by zeros
    static_assert(GF_WAVES * 64 >= 256 * MG, "one reducing thread an output");
    __shared__ float part[2][MG][GF_WAVES][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int kslice = blockIdx.y;
    static_assert(GF_WAVES * GF_KSTEPS * 32 == GF_KSPAN, "a workgroup covers GF_KSPAN of K");
    const int k_lo = kslice * kspan;              // this workgroup's K range starts here
    const int k_hi = (k_lo + kspan < K) ? k_lo + kspan : K;
    const int s0 = wave * ks;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_first = k_lo >> 3, k8_last = (k_hi >> 3) - 1;
    int k8c[GF_KSTEPS];
    bool kok[GF_KSTEPS];
#pragma unroll
    for (int u = 0; u < GF_KSTEPS; ++u) {
        const int k8 = k8_first + (s0 + u) * 4 + q;
        kok[u] = u < ks && k8 <= k8_last;
        k8c[u] = kok[u] ? k8 : (u == 0 ? k8_last : k8c[0]);
    }
    // the first W tile is on its way before anything else (after the X fragments where the activation of
    // two row groups needs the registers meanwhile)
    constexpr bool W_FIRST = !(ACT && MG > 1);
    uint4 a[GF_KSTEPS];
    int tile = blockIdx.x;
    if (W_FIRST && tile < ntiles) {
        const int row = (tile * 16 + r < N) ? tile * 16 + r : N - 1;
        const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)row * ldw);
#pragma unroll
        for (int u = 0; u < GF_KSTEPS; ++u) a[u] = wp[k8c[u]];
    }
    uint4 xf[MG][GF_KSTEPS];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        const bool row_ok = g * 16 + r < M;
        const uint4* xp = reinterpret_cast<const uint4*>(X + (size_t)(row_ok ? g * 16 + r : 0) * lda);
        // with the activation and two row groups the loads come in batches: all of them in flight at once
        // (gate and up of 16 k-steps beside the W tile) would not fit the registers
        constexpr int UB = (ACT && MG > 1) ? 4 : GF_KSTEPS;
#pragma unroll
        for (int u = 0; u < GF_KSTEPS; ++u) {
            if (UB < GF_KSTEPS && u % UB == 0) __builtin_amdgcn_sched_barrier(0);
            uint4 v = xp[k8c[u]];
            if (ACT) {
                const uint4 up = xp[k8c[u] + (K >> 3)];
                const uint32_t gw[4] = {v.x, v.y, v.z, v.w}, uw[4] = {up.x, up.y, up.z, up.w};
                uint32_t o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
                    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
                    // hardware exp2 and reciprocal (about 1 ulp each): the result is rounded to bfloat16 anyway
                    const float s0_ = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g0));
                    const float s1_ = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g1));
                    const f32x2 pr = {g0 * s0_ * u0, g1 * s1_ * u1};
                    o[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2));
                }
                v = make_uint4(o[0], o[1], o[2], o[3]);
            }
            xf[g][u] = (kok[u] && row_ok) ? v : zero;   // zero fragments make the clamped W loads harmless
        }
    }
    if (!W_FIRST && tile < ntiles) {
        __builtin_amdgcn_sched_barrier(0);
        const int row = (tile * 16 + r < N) ? tile * 16 + r : N - 1;
        const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)row * ldw);
#pragma unroll
        for (int u = 0; u < GF_KSTEPS; ++u) a[u] = wp[k8c[u]];
    }
    TC* Cp = C + (size_t)kslice * c_part_stride;
    int buf = 0;
    for (; tile < ntiles; tile += gridDim.x) {
        f32x4 acc[MG];
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < GF_KSTEPS; ++u)
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[g] = gf_mfma(a[u], xf[g][u], acc[g]);
        const int next = tile + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        if (next < ntiles) {   // the next tile's rows are on their way while this one is reduced
            const int row = (next * 16 + r < N) ? next * 16 + r : N - 1;
            const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)row * ldw);
#pragma unroll
            for (int u = 0; u < GF_KSTEPS; ++u) a[u] = wp[k8c[u]];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[buf][g][wave][lane][0]) = acc[g];
        __syncthreads();
        if (threadIdx.x < 256 * MG) {
            const int g = threadIdx.x >> 8, t = threadIdx.x & 255;
            const int e = t & 3, l = t >> 2;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < GF_WAVES; ++w) v += part[buf][g][w][l][e];
            const int n = tile * 16 + (l >> 4) * 4 + e;
            const int m = g * 16 + (l & 15);
            if (n < N && m < M) {
                if (bias != nullptr && kslice == 0) v += to_f32(bias[n]);
                Cp[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
            }
        }
        buf ^= 1;  // the other buffer is free: its readers passed the barrier above one tile ago
    }
}

// Largest K a call takes, given how many parts the caller lets the result be split into.
extern "C" int ilm_gemm_ksplit_max_k(int parts) { return GF_KSPAN * parts; }

// kb > 1: C must be float, [kb][M][ldc] with c_part_stride elements between the parts.
// act != 0: X rows are [gate | up] (2K long) and the product takes silu(gate) * up.
extern "C" int ilm_gemm_ksplit(void* C, int out_dtype, int ldc, long c_part_stride, int kb, const void* W, int ldw,
                               const void* bias, float alpha, int M, int N, int K, const void* X, int lda,
                               int act, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 32 && N > 0 && K > 0, "gemm_ksplit: needs 1 <= M <= 32, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 8 == 0 && ldw % 8 == 0 && ldw >= K && ldc >= N, "gemm_ksplit: K=%d ldw=%d ldc=%d", K, ldw, ldc);
    ILM_REQUIRE(kb >= 1 && K <= ilm_gemm_ksplit_max_k(kb), "gemm_ksplit: K=%d does not fit %d parts of %d", K, kb,
                GF_KSPAN);
    ILM_REQUIRE(kb == 1 || out_dtype == ILM_DTYPE_F32, "gemm_ksplit: partial results are float");
    ILM_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0 && lda % 8 == 0 && lda >= (act ? 2 * K : K),
                "gemm_ksplit: X and W rows must be 16-byte aligned, X rows %d long", act ? 2 * K : K);
    const int ntiles = (N + 15) / 16;
    const int kspan = ((K + kb - 1) / kb + 31) / 32 * 32;   // K spread evenly over the parts
    int gx = ilm_num_cus() / kb;
    if (gx < 1) gx = 1;
    if (gx > ntiles) gx = ntiles;
    dim3 grid(gx, kb);
#define KS_LAUNCH_(WV, KS, MGR, ACT, TC)                                                                       \
    gemm_ksplit_kernel<WV, KS, MGR, ACT, TC><<<grid, WV * 64, 0, stream>>>(                                    \
        (TC*)C, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, N, K, lda, ldw, ldc, alpha, ntiles,      \
        (size_t)c_part_stride, kspan, (kspan / 32 + WV - 1) / WV)
#define KS_LAUNCH(ACT, TC)                                   \
    if (M <= 16) KS_LAUNCH_(16, 8, 1, ACT, TC);              \
    else KS_LAUNCH_(8, 16, 2, ACT, TC)
    if (out_dtype == ILM_DTYPE_BF16) {
        if (act) { KS_LAUNCH(true, bf16); } else { KS_LAUNCH(false, bf16); }
    } else if (out_dtype == ILM_DTYPE_F32) {
        if (act) { KS_LAUNCH(true, float); } else { KS_LAUNCH(false, float); }
    } else {
        ILM_REQUIRE(false, "gemm_ksplit: unknown output dtype %d", out_dtype);
    }
#undef KS_LAUNCH_
#undef KS_LAUNCH
    ILM_LAUNCH_CHECK("gemm_ksplit");
    return 0;
}
