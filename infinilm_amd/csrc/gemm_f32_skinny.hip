// C[M,N] = alpha * (X[M,K] W[N,K]^T + bias) in true 32-bit for few rows of X (M <= 64): the
// projections of a decode step on the 32-bit path, bound by reading W once.
//
// v_mfma_f32_16x16x4_f32 (IEEE float products and sums, no reduced-precision mode) with W rows on the
// A side and tokens on the B side.  A lane loads 16 bytes (4 consecutive k) of its W row and of its
// token's X row and feeds them to four matrix instructions, one per element: instruction j
// reduces over the k values {4 q + j}.  The waves of a workgroup split K into contiguous slices;
// their partial tiles are summed through LDS in wave order.  The order of an output's sum depends on
// K alone (the eight slices, the 16-wide steps inside them, the four instructions of a step), not on
// M, on the batch or on the place of the row in it: rows of any two calls of this kernel agree bit
// for bit.  It is not the ascending-k order of the many-rows kernel (gemm_basic.hip), from which a
// result differs by rounding.
// K must be a multiple of 4 and rows 16-byte aligned.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;

#define FS_UNROLL 4   // 16-wide k-steps whose loads are in flight together, twice over

__device__ __forceinline__ f32x4 fs_mfma(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

#define FS_WAVES 8   // the same for every shape: it fixes the order of the sums

// MG: groups of 16 rows of X; RT: tiles of 16 W rows a workgroup
template <int MG, int RT>
__global__ void __launch_bounds__(FS_WAVES * 64)
gemm_f32_skinny_kernel(float* __restrict__ C, const float* __restrict__ X, const float* __restrict__ W,
                       const float* __restrict__ bias, int M, int N, int K, int lda, int ldw, int ldc, float alpha) {
    __shared__ float part[FS_WAVES][RT][MG][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * (16 * RT);
    const int steps_total = (K + 15) >> 4;
    const int per = (steps_total + FS_WAVES - 1) / FS_WAVES;
    const int s0 = wave * per;
    const int s1 = (s0 + per < steps_total) ? s0 + per : steps_total;
    const int k4_last = (K >> 2) - 1;   // last valid group of 4 elements of a row

    const float4* wp[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int row = (n0 + t * 16 + r < N) ? n0 + t * 16 + r : N - 1;
        wp[t] = reinterpret_cast<const float4*>(W + (size_t)row * ldw);
    }
    const float4* xp[MG];
    bool xok[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        xok[g] = g * 16 + r < M;
        xp[g] = reinterpret_cast<const float4*>(X + (size_t)(xok[g] ? g * 16 + r : 0) * lda);
    }
    f32x4 acc[RT][MG];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Unconditional 16-byte loads from clamped addresses; what lies beyond K, beyond the wave's slice or
    // beyond M is replaced by zeros on the X side.  The chunk after the one being multiplied is on its way.
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 a[2][FS_UNROLL][RT];
    float4 b[2][FS_UNROLL][MG];
#define FS_LOAD(BUF_, S_)                                                          \
    _Pragma("unroll") for (int u = 0; u < FS_UNROLL; ++u) {                        \
        const int k4 = ((S_) + u) * 4 + q;                                         \
        const int k4c = k4 < k4_last ? k4 : k4_last;                               \
        _Pragma("unroll") for (int t = 0; t < RT; ++t) a[BUF_][u][t] = wp[t][k4c]; \
        _Pragma("unroll") for (int g = 0; g < MG; ++g) b[BUF_][u][g] = xp[g][k4c]; \
    }
#define FS_MUL(BUF_, S_)                                                           \
    _Pragma("unroll") for (int u = 0; u < FS_UNROLL; ++u) {                        \
        const int k4 = ((S_) + u) * 4 + q;                                         \
        const bool ok = ((S_) + u < s1) && (k4 <= k4_last);                        \
        _Pragma("unroll") for (int g = 0; g < MG; ++g) {                           \
            const float4 xv = (ok && xok[g]) ? b[BUF_][u][g] : zero;               \
            _Pragma("unroll") for (int t = 0; t < RT; ++t) {                       \
                const float4 wv = a[BUF_][u][t];                                   \
                acc[t][g] = fs_mfma(wv.x, xv.x, acc[t][g]);                        \
                acc[t][g] = fs_mfma(wv.y, xv.y, acc[t][g]);                        \
                acc[t][g] = fs_mfma(wv.z, xv.z, acc[t][g]);                        \
                acc[t][g] = fs_mfma(wv.w, xv.w, acc[t][g]);                        \
            }                                                                      \
        }                                                                          \
    }
    if (s0 < s1) FS_LOAD(0, s0)
    for (int s = s0; s < s1; s += 2 * FS_UNROLL) {
        if (s + FS_UNROLL < s1) FS_LOAD(1, s + FS_UNROLL)
        __builtin_amdgcn_sched_barrier(0);
        FS_MUL(0, s)
        __builtin_amdgcn_sched_barrier(0);
        if (s + 2 * FS_UNROLL < s1) FS_LOAD(0, s + 2 * FS_UNROLL)
        __builtin_amdgcn_sched_barrier(0);
        if (s + FS_UNROLL < s1) FS_MUL(1, s + FS_UNROLL)
        __builtin_amdgcn_sched_barrier(0);
    }
#undef FS_LOAD
#undef FS_MUL
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[wave][t][g][lane][0]) = acc[t][g];
    __syncthreads();
    // acc[t][g][e] of lane (r, q) is output row n0 + t*16 + q*4 + e for token g*16 + r
    for (int idx = threadIdx.x; idx < RT * MG * 64 * 4; idx += FS_WAVES * 64) {
        const int e = idx & 3, l = (idx >> 2) & 63, tg = idx >> 8;
        const int t = tg / MG, g = tg % MG;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < FS_WAVES; ++w) v += part[w][t][g][l][e];
        const int n = n0 + t * 16 + (l >> 4) * 4 + e;
        const int m = g * 16 + (l & 15);
        if (n < N && m < M) {
            if (bias != nullptr) v += bias[n];
            C[(size_t)m * ldc + n] = alpha * v;
        }
    }
}

extern "C" int ilm_gemm_f32_skinny(void* C, const void* X, const void* W, const void* bias, int M, int N, int K,
                                   int lda, int ldw, int ldc, float alpha, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_f32_skinny: needs 1 <= M <= 64, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && lda >= K && ldw >= K && ldc >= N,
                "gemm_f32_skinny: K=%d lda=%d ldw=%d ldc=%d", K, lda, ldw, ldc);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_f32_skinny: operands must be 16-byte aligned");
    const int mg = (M + 15) / 16;
#define FS_CASE(MG_, RT_)                                                                                       \
    gemm_f32_skinny_kernel<MG_, RT_><<<(N + 16 * RT_ - 1) / (16 * RT_), FS_WAVES * 64, 0, stream>>>(            \
        (float*)C, (const float*)X, (const float*)W, (const float*)bias, M, N, K, lda, ldw, ldc, alpha)
    // two tiles a workgroup where W is tall enough to still fill the chip: an X fragment read once serves both
    const bool tall = N >= 16384;
    switch (mg) {
        case 1: if (tall) FS_CASE(1, 2); else FS_CASE(1, 1); break;
        case 2: if (tall) FS_CASE(2, 2); else FS_CASE(2, 1); break;
        case 3: FS_CASE(3, 1); break;
        default: FS_CASE(4, 1); break;
    }
#undef FS_CASE
    ILM_LAUNCH_CHECK("gemm_f32_skinny");
    return 0;
}
