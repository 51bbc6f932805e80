// The fused q/k/v projection with the rotation of q and k and the write of k and v into the paged cache
// in its epilogue, for 17 to 64 rows of X (bfloat16): decode steps of many requests, where X no longer
// fits a wave's registers.
//
// As in gemm_qkv_rope.hip a workgroup takes a run of up to 16 rotation pairs (rows i and i + d/2 of a head
// slot) and multiplies two 16-row tiles of W, the pairs' first and second rows, on v_mfma_f32_16x16x32_bf16;
// the 8 waves split K evenly and their partial tiles meet in LDS, where the thread that reduces output
// (m, n) of the first tile also reduces (m, n) of the second, rotates the pair by the token's position and
// stores it.  Unlike there, a wave does not keep its X fragments: it streams them beside the W fragments, a
// chunk of QW_CH k-steps ahead of the one it multiplies.  W comes from memory once; X (at most 64 rows) is
// read by every workgroup, from the L2s: the price of one owner an output without a pass through LDS, paid
// where W has so few rows (some thousand) that a workgroup cannot own enough of them to share an X tile.
// Needs the whole head rotated (rotary dim = head dim) and head dims in steps of 32.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define QW_WAVES 8

__device__ __forceinline__ f32x4 qw_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// round to bfloat16 and back: the unfused path stores the projection in bfloat16 before it rotates
__device__ __forceinline__ float qw_round(float v) { return to_f32(from_f32<bf16>(v)); }

// MG: groups of 16 rows of X; CH: k-steps of 32 a chunk
template <int MG, int CH>
__global__ void __launch_bounds__(QW_WAVES * 64)
gemm_qkv_rope_wide_kernel(bf16* __restrict__ Q, const bf16* __restrict__ X, const bf16* __restrict__ W,
                          const bf16* __restrict__ bias, int M, int K, int lda, int ldw, int ldq,
                          const int* __restrict__ pos, const float* __restrict__ cosT, const float* __restrict__ sinT,
                          bf16* __restrict__ kc, bf16* __restrict__ vc, const int* __restrict__ slots, int nh, int nkv,
                          int d, int page, int n_units, int pairs_per_unit, int ks) {
    __shared__ float part[2][MG][QW_WAVES][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int half = d >> 1;
    const int total_pairs = (nh + 2 * nkv) * half;
    const int k8_last = (K >> 3) - 1;
    const int s0 = wave * ks, s1 = s0 + ks;   // the wave's k-steps (beyond K: zeros)
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);

    const uint4* xp[MG];
    bool xok[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        xok[g] = g * 16 + r < M;
        xp[g] = reinterpret_cast<const uint4*>(X + (size_t)(xok[g] ? g * 16 + r : 0) * lda);
    }
    for (int unit = blockIdx.x; unit < n_units; unit += gridDim.x) {
        // this lane's W rows: pair p0 + r of the run, first and second row (lanes beyond the run repeat its last pair)
        const int p0 = unit * pairs_per_unit;
        const int np = total_pairs - p0 < pairs_per_unit ? total_pairs - p0 : pairs_per_unit;
        const int pr = p0 + (r < np ? r : np - 1);
        const int row0 = (pr / half) * d + pr % half;
        const uint4* wp0 = reinterpret_cast<const uint4*>(W + (size_t)row0 * ldw);
        const uint4* wp1 = reinterpret_cast<const uint4*>(W + (size_t)(row0 + half) * ldw);

        f32x4 acc[2][MG];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};
        uint4 a[2][CH][2], b[2][CH][MG];
        // unconditional loads from clamped addresses; what lies beyond K is replaced by zeros on the X side
#define QW_LOAD(BUF_, S_)                                                          \
        _Pragma("unroll") for (int u = 0; u < CH; ++u) {                           \
            const int k8 = ((S_) + u) * 4 + q;                                     \
            const int k8c = k8 < k8_last ? k8 : k8_last;                           \
            a[BUF_][u][0] = wp0[k8c];                                              \
            a[BUF_][u][1] = wp1[k8c];                                              \
            _Pragma("unroll") for (int g = 0; g < MG; ++g) b[BUF_][u][g] = xp[g][k8c]; \
        }
#define QW_MUL(BUF_, S_)                                                           \
        _Pragma("unroll") for (int u = 0; u < CH; ++u) {                           \
            const int k8 = ((S_) + u) * 4 + q;                                     \
            const bool ok = ((S_) + u < s1) && k8 <= k8_last;                      \
            _Pragma("unroll") for (int g = 0; g < MG; ++g) {                       \
                const uint4 xv = (ok && xok[g]) ? b[BUF_][u][g] : zero;            \
                acc[0][g] = qw_mfma(a[BUF_][u][0], xv, acc[0][g]);                 \
                acc[1][g] = qw_mfma(a[BUF_][u][1], xv, acc[1][g]);                 \
            }                                                                      \
        }
        QW_LOAD(0, s0)
        for (int s = s0; s < s1; s += 2 * CH) {
            if (s + CH < s1) QW_LOAD(1, s + CH)
            __builtin_amdgcn_sched_barrier(0);
            QW_MUL(0, s)
            __builtin_amdgcn_sched_barrier(0);
            if (s + 2 * CH < s1) QW_LOAD(0, s + 2 * CH)
            __builtin_amdgcn_sched_barrier(0);
            if (s + CH < s1) QW_MUL(1, s + CH)
            __builtin_amdgcn_sched_barrier(0);
        }
#undef QW_LOAD
#undef QW_MUL
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[t][g][wave][lane][0]) = acc[t][g];
        __syncthreads();
        // acc[t][g][e] of lane (r, q): pair slot 4 q + e of the run, row g * 16 + r of X
        for (int et = threadIdx.x; et < 256 * MG; et += QW_WAVES * 64) {
            const int eg = et >> 8, e = et & 3, l = (et & 255) >> 2;
            const int m = eg * 16 + (l & 15), nl = (l >> 4) * 4 + e;
            const int pair = p0 + nl;
            if (m >= M || nl >= np) continue;
            const int hs = pair / half, i0 = pair % half;   // head slot, dim within its first half
            float val[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                float v = 0.f;
#pragma unroll
                for (int w = 0; w < QW_WAVES; ++w) v += part[t][eg][w][l][e];
                if (bias != nullptr) v += to_f32(bias[hs * d + i0 + t * half]);
                val[t] = qw_round(v);
            }
            const int slot = slots != nullptr ? slots[m] : -1;
            if (hs < nh + nkv) {
                const int p_m = pos[m];
                const float cs = cosT[(size_t)p_m * half + i0], sn = sinT[(size_t)p_m * half + i0];
                const float ra = val[0] * cs - val[1] * sn;
                const float rb = val[1] * cs + val[0] * sn;
                if (hs < nh) {
                    bf16* dst = Q + (size_t)m * ldq + (size_t)hs * d + i0;
                    dst[0] = from_f32<bf16>(ra);
                    dst[half] = from_f32<bf16>(rb);
                } else if (slot >= 0) {
                    bf16* dst = kc + (((size_t)(slot / page) * nkv + (hs - nh)) * page + (slot % page)) * d + i0;
                    dst[0] = from_f32<bf16>(ra);
                    dst[half] = from_f32<bf16>(rb);
                }
            } else if (slot >= 0) {
                // values are cached transposed, [pages, nkv, d, page]
                bf16* dst = vc + ((size_t)(slot / page) * nkv + (hs - nh - nkv)) * d * page + (slot % page);
                dst[(size_t)i0 * page] = from_f32<bf16>(val[0]);
                dst[(size_t)(i0 + half) * page] = from_f32<bf16>(val[1]);
            }
        }
        __syncthreads();   // the next unit's partial tiles go to the same LDS
    }
}

// As ilm_gemm_qkv_rope, for 17 <= M <= 64.  `pairs_per_unit`: 0 = chosen here (16, or fewer where that gives
// every compute unit a run).
extern "C" int ilm_gemm_qkv_rope_wide(void* Q, int ldq, const void* X, int lda, const void* W, int ldw, const void* bias,
                                      int M, int K, const void* pos, const void* cosT, const void* sinT, void* kc,
                                      void* vc, const void* slots, int nh, int nkv, int d, int page, int pairs_per_unit,
                                      hipStream_t stream) {
    ILM_REQUIRE(M > 16 && M <= 64 && K > 0 && nh > 0 && nkv >= 0, "gemm_qkv_rope_wide: needs 17 <= M <= 64, got M=%d K=%d", M, K);
    ILM_REQUIRE(d > 0 && d % 32 == 0, "gemm_qkv_rope_wide: head size %d is not a multiple of 32", d);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldq >= nh * d,
                "gemm_qkv_rope_wide: K=%d lda=%d ldw=%d ldq=%d", K, lda, ldw, ldq);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_qkv_rope_wide: operands must be 16-byte aligned");
    ILM_REQUIRE(slots == nullptr || (page > 0 && kc != nullptr && vc != nullptr), "gemm_qkv_rope_wide: cache missing");
    ILM_REQUIRE(pairs_per_unit >= 0 && pairs_per_unit <= 16, "gemm_qkv_rope_wide: %d pairs a run", pairs_per_unit);
    const int ksteps = (K + 31) / 32;
    const int total_pairs = (nh + 2 * nkv) * (d / 2);
    int ppu = pairs_per_unit;
    if (ppu == 0) {
        const int cus = ilm_num_cus();
        ppu = (total_pairs + cus - 1) / cus;
        if (ppu > 16) ppu = 16;
        if (ppu < 8) ppu = 8;
    }
    const int n_units = (total_pairs + ppu - 1) / ppu;
    const int cap = 2 * ilm_num_cus();
    const int grid = n_units < cap ? n_units : cap;
    const int ks = (ksteps + QW_WAVES - 1) / QW_WAVES;
#define QW_CASE(MG_, CH_)                                                                                       \
    gemm_qkv_rope_wide_kernel<MG_, CH_><<<grid, QW_WAVES * 64, 0, stream>>>(                                    \
        (bf16*)Q, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, K, lda, ldw, ldq, (const int*)pos,      \
        (const float*)cosT, (const float*)sinT, (bf16*)kc, (bf16*)vc, (const int*)slots, nh, nkv, d, page,      \
        n_units, ppu, ks)
    switch ((M + 15) / 16) {
        case 2: QW_CASE(2, 4); break;
        case 3: QW_CASE(3, 4); break;
        default: QW_CASE(4, 3); break;
    }
#undef QW_CASE
    ILM_LAUNCH_CHECK("gemm_qkv_rope_wide");
    return 0;
}
