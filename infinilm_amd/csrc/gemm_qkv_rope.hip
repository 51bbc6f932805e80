// The fused q/k/v projection of a decode step (at most 32 rows of X, bfloat16) with the rotation of
// q and k and the write of k and v into the paged cache in its epilogue: one kernel instead of
// two between the norm and the attention.
//
// The product is the resident few-rows one (X fragments in registers, W streamed once on
// v_mfma_f32_16x16x32_bf16, K split over the waves and reduced through LDS).  Rows i and i + d/2 of
// a head slot (q head, k head or v head) form a pair; a workgroup takes a run of up to 16
// consecutive pairs and multiplies two 16-row tiles of W: the pairs' first rows and their second
// rows.  The thread that reduces output (m, n) of the first tile also reduces (m, n) of the
// second, so it holds a pair in registers, rotates it by the token's position and stores it: q
// into the output rows, k into the token's cache slot; v pairs take the same path without
// rotation into the transposed value cache.  The run length is chosen so that every compute unit
// gets one run (9 pairs = 18 rows at the 8B shape: no second round for a few leftover tiles).
// Needs the whole head rotated (rotary dim = head dim) and head dims in steps of 32.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ f32x4 qr_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// round to bfloat16 and back: the unfused path stores the projection in bfloat16 before it rotates
__device__ __forceinline__ float qr_round(float v) { return to_f32(from_f32<bf16>(v)); }

// MG: groups of 16 rows of X whose fragments a wave keeps (two groups: 8 waves under 256 registers)
template <int WAVES, int KSTEPS, int MG>
__global__ void __launch_bounds__(WAVES * 64)
gemm_qkv_rope_kernel(bf16* __restrict__ Q, const bf16* __restrict__ X, const bf16* __restrict__ W,
                     const bf16* __restrict__ bias, int M, int K, int lda, int ldw, int ldq,
                     const int* __restrict__ pos, const float* __restrict__ cosT, const float* __restrict__ sinT,
                     bf16* __restrict__ kc, bf16* __restrict__ vc, const int* __restrict__ slots, int nh, int nkv,
                     int d, int page, int n_units, int pairs_per_unit, int ks) {
    // ks <= KSTEPS: k-steps a wave really takes (K spread evenly over the waves); its other slots load
    // its first address again (a cache hit, no branch around the loads) and multiply by zeros
    static_assert(WAVES * 64 >= 256 * MG, "one reducing thread an output");
    __shared__ float part[2][MG][WAVES][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int s0 = wave * ks;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (K >> 3) - 1;
    const int half = d >> 1;
    uint4 xf[MG][KSTEPS];
    int k8c[KSTEPS];
    bool kok[KSTEPS];
#pragma unroll
    for (int u = 0; u < KSTEPS; ++u) {
        const int k8 = (s0 + u) * 4 + q;
        kok[u] = u < ks && k8 <= k8_last;
        k8c[u] = kok[u] ? k8 : (u == 0 ? k8_last : k8c[0]);
    }
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        const int row = g * 16 + r;
        const uint4* xp = reinterpret_cast<const uint4*>(X + (size_t)(row < M ? row : 0) * lda);
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u) {
            const uint4 v = xp[k8c[u]];
            xf[g][u] = (kok[u] && row < M) ? v : zero;   // zero fragments make the clamped W loads harmless
        }
    }
    // pair p: rows hs*d + i and hs*d + i + d/2 with hs = p / (d/2), i = p % (d/2)
    const int total_pairs = (nh + 2 * nkv) * half;
    auto first_row = [&](int pair) -> int { return (pair / half) * d + pair % half; };
    // this lane's W row of a unit's tile (0: first rows, 1: second rows); lanes beyond the run repeat its last pair
    auto tile_row = [&](int u, int half_idx) -> int {
        const int p0 = u * pairs_per_unit;
        const int np = total_pairs - p0 < pairs_per_unit ? total_pairs - p0 : pairs_per_unit;
        return first_row(p0 + (r < np ? r : np - 1)) + half_idx * half;
    };
    uint4 a[KSTEPS];
    int unit = blockIdx.x;
    if (unit < n_units) {
        const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)tile_row(unit, 0) * ldw);
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
    }
    // the epilogue thread's output: row m, pair slot nl of the run
    const int et = threadIdx.x < 256 * MG ? threadIdx.x : 0;
    const int eg = et >> 8, e = et & 3, l = (et & 255) >> 2;
    const int m = eg * 16 + (l & 15), nl = (l >> 4) * 4 + e;
    const bool row_writer = threadIdx.x < 256 * MG && m < M;
    const int p_m = row_writer ? pos[m] : 0;
    const int slot = (row_writer && slots != nullptr) ? slots[m] : -1;
    int buf = 0;
    for (; unit < n_units; unit += gridDim.x) {
        const int pair = unit * pairs_per_unit + nl;
        const bool writer = row_writer && nl < pairs_per_unit && pair < total_pairs;
        const int hs = writer ? pair / half : 0, i0 = writer ? pair % half : 0;   // head slot, dim within its first half
        float cs = 1.f, sn = 0.f;
        if (writer && hs < nh + nkv) {   // on their way while the products run
            cs = cosT[(size_t)p_m * half + i0];
            sn = sinT[(size_t)p_m * half + i0];
        }
        float val[2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            f32x4 acc[MG];
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < KSTEPS; ++u)
#pragma unroll
                for (int g = 0; g < MG; ++g) acc[g] = qr_mfma(a[u], xf[g][u], acc[g]);
            // the next tile's rows are on their way while this one is reduced
            const int nu = hf == 0 ? unit : unit + gridDim.x;
            __builtin_amdgcn_sched_barrier(0);
            if (nu < n_units) {
                const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)tile_row(nu, hf == 0 ? 1 : 0) * ldw);
#pragma unroll
                for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[buf][g][wave][lane][0]) = acc[g];
            __syncthreads();
            float v = 0.f;
            if (threadIdx.x < 256 * MG) {
#pragma unroll
                for (int w = 0; w < WAVES; ++w) v += part[buf][eg][w][l][e];
                if (bias != nullptr && writer) v += to_f32(bias[hs * d + i0 + hf * half]);
            }
            val[hf] = qr_round(v);
            buf ^= 1;  // the other buffer is free: its readers passed the barrier above one tile ago
        }
        if (!writer) continue;
        if (hs < nh + nkv) {
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
}

// Q [M, ldq] receives the rotated query heads; k (rotated) and v go to the cache slots (slots may be
// null: nothing is cached).  W [(nh + 2 nkv) d, ldw] holds the q, k, v rows in this order.
extern "C" int ilm_gemm_qkv_rope(void* Q, int ldq, const void* X, int lda, const void* W, int ldw, const void* bias,
                                 int M, int K, const void* pos, const void* cosT, const void* sinT, void* kc, void* vc,
                                 const void* slots, int nh, int nkv, int d, int page, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 32 && K > 0 && nh > 0 && nkv >= 0, "gemm_qkv_rope: needs 1 <= M <= 32, got M=%d K=%d", M, K);
    ILM_REQUIRE(d > 0 && d % 32 == 0, "gemm_qkv_rope: head size %d is not a multiple of 32", d);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldq >= nh * d,
                "gemm_qkv_rope: K=%d lda=%d ldw=%d ldq=%d", K, lda, ldw, ldq);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_qkv_rope: operands must be 16-byte aligned");
    ILM_REQUIRE(slots == nullptr || (page > 0 && kc != nullptr && vc != nullptr), "gemm_qkv_rope: cache missing");
    const int ksteps = (K + 31) / 32;
    ILM_REQUIRE(ksteps <= (M <= 16 ? 16 * 16 : 8 * 16), "gemm_qkv_rope: K=%d is beyond %d", K, M <= 16 ? 8192 : 4096);
    // runs of pairs: one a compute unit where that gives at most 16 pairs a run, else runs of 16 in rounds
    const int total_pairs = (nh + 2 * nkv) * (d / 2);
#define QR_CASE(WV, KS, MGR)                                                                                   \
    {                                                                                                          \
        const int cap = ilm_num_cus() * ((WV == 16 || (MGR == 2 && KS >= 12)) ? 1 : 2);                         \
        int ppu = (total_pairs + cap - 1) / cap;                                                               \
        if (ppu > 16) ppu = 16;                                                                                \
        const int n_units = (total_pairs + ppu - 1) / ppu;                                                     \
        const int grid = n_units < cap ? n_units : cap;                                                        \
        gemm_qkv_rope_kernel<WV, KS, MGR><<<grid, WV * 64, 0, stream>>>(                                            \
            (bf16*)Q, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, K, lda, ldw, ldq, (const int*)pos, \
            (const float*)cosT, (const float*)sinT, (bf16*)kc, (bf16*)vc, (const int*)slots, nh, nkv, d, page, \
            n_units, ppu, (ksteps + WV - 1) / WV);                                                             \
    }
    if (M > 16) {
        if (ksteps <= 8 * 4) QR_CASE(8, 4, 2)
        else if (ksteps <= 8 * 8) QR_CASE(8, 8, 2)
        else if (ksteps <= 8 * 12) QR_CASE(8, 12, 2)
        else QR_CASE(8, 16, 2)
    }
    else if (ksteps <= 8 * 4) QR_CASE(8, 4, 1)
    else if (ksteps <= 8 * 8) QR_CASE(8, 8, 1)
    else if (ksteps <= 8 * 12) QR_CASE(8, 12, 1)   // (a width like 2304: 9 of 12 slots a wave instead of 5 of 8 in 16 waves)
    else if (ksteps <= 16 * 8) QR_CASE(16, 8, 1)
    else if (ksteps <= 16 * 12) QR_CASE(16, 12, 1)
    else QR_CASE(16, 16, 1)
#undef QR_CASE
    ILM_LAUNCH_CHECK("gemm_qkv_rope");
    return 0;
}
