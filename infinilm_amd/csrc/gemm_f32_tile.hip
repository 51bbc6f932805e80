// C[M,N] = alpha * (X[M,K] W[N,K]^T + bias) in true 32-bit for many rows of X (portions of prompts on the
// 32-bit path): tiles of 128 x 128 outputs on v_mfma_f32_16x16x4_f32 (IEEE float products and sums, no
// reduced-precision mode), operands staged through LDS.
//
// The order of an output's sum is that of the few-rows kernel (gemm_f32_skinny.hip), so a row of X gives
// the same bits whether it comes alone, among 64 or among 2,048 rows: K is walked in steps of 16 (a lane's 16
// bytes feed four instructions, instruction e reducing over k = 16 s + 4 q + e), the steps fall into eight
// contiguous slices of ceil(steps / 8) steps, each slice is summed from zero, and the eight slice sums are
// added in ascending order.  (There the slices belong to eight waves and meet in LDS; here one wave walks
// all of them and adds a slice's sum to its total when the next slice begins.)
// K must be a multiple of 4 and rows 16-byte aligned.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;

#define FT_BM 128        // rows of X a workgroup
#define FT_BN 128        // rows of W a workgroup
#define FT_BK 32         // k a stage: two steps of 16
#define FT_LD 36         // floats a row of a stage in LDS (32 + 4: a wave's 16-byte reads fall on distinct banks)
#define FT_SLICES 8      // as gemm_f32_skinny's waves

__device__ __forceinline__ f32x4 ft_mfma(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

__global__ void __launch_bounds__(256)
gemm_f32_tile_kernel(float* __restrict__ C, const float* __restrict__ X, const float* __restrict__ W,
                     const float* __restrict__ bias, int M, int N, int K, int lda, int ldw, int ldc, float alpha,
                     int m_tiles, int n_tiles, int vec_store) {
    __shared__ __align__(16) float Ws[2][FT_BN][FT_LD];
    __shared__ __align__(16) float Xs[2][FT_BM][FT_LD];
    // Workgroups go to the 8 XCDs round-robin: those of one XCD take the m tiles of one n tile one after the
    // other, so a tile of W is fetched into one L2 only.
    int mt, nt;
    {
        const int id = blockIdx.x, total = m_tiles * n_tiles;
        const int full = (n_tiles / 8) * 8 * m_tiles;   // n tiles in whole rounds of 8
        if (id < full) {
            const int xcd = id & 7, local = id >> 3;
            mt = local % m_tiles;
            nt = (local / m_tiles) * 8 + xcd;
        } else {
            const int rest = id - full;
            mt = rest % m_tiles;
            nt = (n_tiles / 8) * 8 + rest / m_tiles;
        }
        (void)total;
    }
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, q = lane >> 4;
    const int n0 = nt * FT_BN, m0 = mt * FT_BM;
    const int wn = (wave & 1) * 64, wm = (wave >> 1) * 64;   // the wave's 64 x 64 outputs inside the tile

    const int steps_total = (K + 15) >> 4;
    const int per = (steps_total + FT_SLICES - 1) / FT_SLICES;
    const int stages = (K + FT_BK - 1) / FT_BK;
    const int k4_last = (K >> 2) - 1;

    // a thread stages 16 bytes of 4 rows of each operand: row tid / 8 + 32 i, k offset 4 (tid % 8)
    const int lrow = tid >> 3, lk4 = tid & 7;
    const float4* wsrc[4];
    const float4* xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int wr = n0 + lrow + 32 * i, xr = m0 + lrow + 32 * i;
        wsrc[i] = reinterpret_cast<const float4*>(W + (size_t)(wr < N ? wr : N - 1) * ldw);
        xsrc[i] = reinterpret_cast<const float4*>(X + (size_t)(xr < M ? xr : M - 1) * lda);
    }
    float4 wreg[4], xreg[4];
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#define FT_FETCH(ST_)                                                            \
    {                                                                            \
        const int k4 = (ST_) * (FT_BK / 4) + lk4;                                \
        const int k4c = k4 < k4_last ? k4 : k4_last;                             \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                          \
            wreg[i] = wsrc[i][k4c];                                              \
            xreg[i] = xsrc[i][k4c];                                              \
        }                                                                        \
        if (k4 > k4_last) {   /* beyond K: zeros on the X side, as the few-rows kernel has them */ \
            _Pragma("unroll") for (int i = 0; i < 4; ++i) xreg[i] = zero;        \
        }                                                                        \
    }
#define FT_STORE(BUF_)                                                                                   \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                                      \
        *reinterpret_cast<float4*>(&Ws[BUF_][lrow + 32 * i][4 * lk4]) = wreg[i];                         \
        *reinterpret_cast<float4*>(&Xs[BUF_][lrow + 32 * i][4 * lk4]) = xreg[i];                         \
    }

    f32x4 acc[4][4], total[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};
            total[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};
        }

    FT_FETCH(0)
    FT_STORE(0)
    __syncthreads();
    for (int st = 0; st < stages; ++st) {
        const int buf = st & 1;
        if (st + 1 < stages) FT_FETCH(st + 1)
#pragma unroll
        for (int hs = 0; hs < 2; ++hs) {
            const int s = 2 * st + hs;
            if (s < steps_total) {
                if (s > 0 && s % per == 0) {   // a slice ends: its sum joins the total, the next starts from zero
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            total[t][g] += acc[t][g];
                            acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};
                        }
                }
                float4 a[4], b[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) a[t] = *reinterpret_cast<const float4*>(&Ws[buf][wn + 16 * t + r][16 * hs + 4 * q]);
#pragma unroll
                for (int g = 0; g < 4; ++g) b[g] = *reinterpret_cast<const float4*>(&Xs[buf][wm + 16 * g + r][16 * hs + 4 * q]);
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        acc[t][g] = ft_mfma(a[t].x, b[g].x, acc[t][g]);
                        acc[t][g] = ft_mfma(a[t].y, b[g].y, acc[t][g]);
                        acc[t][g] = ft_mfma(a[t].z, b[g].z, acc[t][g]);
                        acc[t][g] = ft_mfma(a[t].w, b[g].w, acc[t][g]);
                    }
            }
        }
        if (st + 1 < stages) {
            FT_STORE(buf ^ 1)
        }
        __syncthreads();
    }
#undef FT_FETCH
#undef FT_STORE
    // acc[t][g][e] of lane (r, q): output row m0 + wm + 16 g + r, column n0 + wn + 16 t + 4 q + e
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int m = m0 + wm + 16 * g + r;
        if (m >= M) continue;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int n = n0 + wn + 16 * t + 4 * q;
            if (n >= N) continue;
            f32x4 v = total[t][g] + acc[t][g];
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x = v[e];
                if (bias != nullptr && n + e < N) x += bias[n + e];
                o[e] = alpha * x;
            }
            float* dst = C + (size_t)m * ldc + n;
            if (vec_store && n + 3 < N) {
                *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) dst[e] = o[e];
            }
        }
    }
}

extern "C" int ilm_gemm_f32_tile(void* C, const void* X, const void* W, const void* bias, int M, int N, int K,
                                 int lda, int ldw, int ldc, float alpha, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_f32_tile: bad sizes M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && lda >= K && ldw >= K && ldc >= N,
                "gemm_f32_tile: K=%d lda=%d ldw=%d ldc=%d", K, lda, ldw, ldc);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_f32_tile: operands must be 16-byte aligned");
    const int m_tiles = (M + FT_BM - 1) / FT_BM, n_tiles = (N + FT_BN - 1) / FT_BN;
    ILM_REQUIRE((long long)m_tiles * n_tiles < (1ll << 31), "gemm_f32_tile: too many tiles");
    const int vec_store = (ldc % 4 == 0 && ((uintptr_t)C & 15) == 0) ? 1 : 0;
    gemm_f32_tile_kernel<<<m_tiles * n_tiles, 256, 0, stream>>>((float*)C, (const float*)X, (const float*)W,
                                                               (const float*)bias, M, N, K, lda, ldw, ldc, alpha, m_tiles,
                                                               n_tiles, vec_store);
    ILM_LAUNCH_CHECK("gemm_f32_tile");
    return 0;
}
