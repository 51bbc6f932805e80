// C[M,N] = alpha * (X[M,K] W[N,K]^T + bias) for few rows of X (M <= 64), bfloat16 in, float
// accumulation: the decode-side projection, bound by reading W once from HBM.
//
// v_mfma_f32_16x16x32_bf16 with W rows on the A side and tokens on the B side: one accumulator is
// 16 outputs x 16 tokens.  The waves of a workgroup split K into contiguous slices and stream
// their slice of the workgroup's W rows straight from global memory into MFMA operands; the
// partial tiles are summed through LDS in wave order, so the result is deterministic.
//
// Two kernels:
//  * stream:  RT tiles of 16 W rows per workgroup, up to 4 token groups; the X fragments are
//             re-read from L2 for every workgroup.  Any K (multiple of 8), any M <= 64.
//  * resident (M <= 16 and K <= 8192, or M <= 32 and K <= 4096): each wave keeps the X fragments of its
//             K slice in registers and the workgroup walks over W row tiles, prefetching the next
//             tile's rows while the current one is reduced; X is read once per workgroup.
// K must be a multiple of 8 (16-byte loads); rows of X and W must be 16-byte aligned.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;


__device__ __forceinline__ f32x4 mfma16(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <int WAVES, int MG, int RT, int UNROLL, typename TC>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_stream_kernel(TC* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W,
                          const bf16* __restrict__ bias, int M, int N, int K, int lda, int ldw, int ldc,
                          float alpha) {
    __shared__ float part[WAVES][RT][MG][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * (16 * RT);
    const int steps_total = (K + 31) >> 5;
    const int per = (steps_total + WAVES - 1) / WAVES;
    const int s0 = wave * per;
    const int s1 = (s0 + per < steps_total) ? s0 + per : steps_total;

    const uint4* wp[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int row = (n0 + t * 16 + r < N) ? n0 + t * 16 + r : N - 1;
        wp[t] = reinterpret_cast<const uint4*>(W + (size_t)row * ldw);
    }
    const uint4* xp[MG];
    bool xok[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        xok[g] = g * 16 + r < M;
        xp[g] = reinterpret_cast<const uint4*>(X + (size_t)(xok[g] ? g * 16 + r : 0) * lda);
    }
    f32x4 acc[RT][MG];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Loads are unconditional 16-byte loads from clamped (always valid) addresses; what lies beyond K,
    // beyond this wave's slice or beyond M is replaced by zeros afterwards.  (A conditional load
    // would be split into four 4-byte loads behind branches.)  The chunk after the one being
    // multiplied is already on its way.
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (K >> 3) - 1;
    uint4 a[2][UNROLL][RT];
    uint4 b[2][UNROLL][MG];
    auto load_chunk = [&](int s, int buf) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k8 = (s + u) * 4 + q;  // index of this lane's group of 8 elements
            const int k8c = k8 < k8_last ? k8 : k8_last;
#pragma unroll
            for (int t = 0; t < RT; ++t) a[buf][u][t] = wp[t][k8c];
#pragma unroll
            for (int g = 0; g < MG; ++g) b[buf][u][g] = xp[g][k8c];
        }
    };
    auto mul_chunk = [&](int s, int buf) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k8 = (s + u) * 4 + q;
            const bool ok = (s + u < s1) && (k8 <= k8_last);
#pragma unroll
            for (int t = 0; t < RT; ++t)
#pragma unroll
                for (int g = 0; g < MG; ++g)
                    acc[t][g] = mfma16(ok ? a[buf][u][t] : zero, xok[g] ? b[buf][u][g] : zero, acc[t][g]);
        }
    };
    if (s0 < s1) load_chunk(s0, 0);
    for (int s = s0; s < s1; s += 2 * UNROLL) {
        if (s + UNROLL < s1) load_chunk(s + UNROLL, 1);
        __builtin_amdgcn_sched_barrier(0);
        mul_chunk(s, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (s + 2 * UNROLL < s1) load_chunk(s + 2 * UNROLL, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (s + UNROLL < s1) mul_chunk(s + UNROLL, 1);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g)
            *reinterpret_cast<f32x4*>(&part[wave][t][g][lane][0]) = acc[t][g];
    __syncthreads();
    // acc[t][g][e] of lane (r, q) is output row n0 + t*16 + q*4 + e for token g*16 + r
    for (int idx = threadIdx.x; idx < RT * MG * 64 * 4; idx += WAVES * 64) {
        const int e = idx & 3, l = (idx >> 2) & 63, tg = idx >> 8;
        const int t = tg / MG, g = tg % MG;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) v += part[w][t][g][l][e];
        const int n = n0 + t * 16 + (l >> 4) * 4 + e;
        const int m = g * 16 + (l & 15);
        if (n < N && m < M) {
            if (bias != nullptr) v += to_f32(bias[n]);
            C[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
        }
    }
}

// M <= 16 MG.  WAVES waves of KSTEPS k-steps (32 elements each) cover K; the X fragments of MG groups
// of 16 rows stay in registers, so a W fragment read once serves MG matrix instructions.
template <int WAVES, int KSTEPS, int MG, typename TC>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_resident_kernel(TC* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W,
                            const bf16* __restrict__ bias, int M, int N, int K, int lda, int ldw, int ldc,
                            float alpha, int ntiles, int ks) {
    // ks <= KSTEPS: k-steps a wave really takes (K spread evenly over the waves); its other slots load
    // its first address again (a cache hit, no branch around the loads) and multiply by zeros
    static_assert(WAVES * 64 >= 256 * MG, "one reducing thread an output");
    __shared__ float part[2][MG][WAVES][64][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int s0 = wave * ks;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (K >> 3) - 1;
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
            // zero fragments beyond K or beyond M make the clamped W loads harmless
            xf[g][u] = (kok[u] && row < M) ? v : zero;
        }
    }
    uint4 a[KSTEPS];
    int tile = blockIdx.x;
    if (tile < ntiles) {
        const int row = (tile * 16 + r < N) ? tile * 16 + r : N - 1;
        const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)row * ldw);
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
    }
    int buf = 0;
    for (; tile < ntiles; tile += gridDim.x) {
        f32x4 acc[MG];
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u)
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[g] = mfma16(a[u], xf[g][u], acc[g]);
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
        if (threadIdx.x < 256 * MG) {
            const int g = threadIdx.x >> 8, t = threadIdx.x & 255;
            const int e = t & 3, l = t >> 2;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) v += part[buf][g][w][l][e];
            const int n = tile * 16 + (l >> 4) * 4 + e;
            const int m = g * 16 + (l & 15);
            if (n < N && m < M) {
                if (bias != nullptr) v += to_f32(bias[n]);
                C[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
            }
        }
        buf ^= 1;  // the other buffer is free: its readers passed the barrier above one tile ago
    }
}

// 1 / sqrt(mean(r^2) + eps) of a row from the partial sums of squares a producer left (gemm_tail.hip:
// SS[tile][32]), for a product whose X is that producer's r * w, not yet divided: the division is one
// number a row and is applied to the sums in the epilogue.  In three pieces, so that nothing waits:
//   SK_SCALE_LOAD   before the main loop: a thread takes four rows (one 16-byte load a tile) of the tiles
//                   c, c + C, c + 2C, ... (C = threads / (4 MG) chunks); the loads fly with the first W tile
//   SK_SCALE_PUT    in the first round, before the barrier the reduction of the tile has anyway: the chunks of
//                   a wave are added by shuffles, the wave's sums go to LDS `ssr[WAVES][32]`
//   SK_SCALE_GET    after that barrier: the waves' sums in wave order
// The order of the sum depends on the number of tiles alone.
#define SK_SCALE_LOAD(SS_, TILES_)                                                                \
    float4 ss_sum = make_float4(0.f, 0.f, 0.f, 0.f);                                              \
    if ((SS_) != nullptr) {                                                                       \
        constexpr int Q_ = 4 * MG, C_ = WAVES * 64 / Q_;                                          \
        const float4* sp = reinterpret_cast<const float4*>(SS_) + threadIdx.x % Q_;               \
        int tl = threadIdx.x / Q_;                                                                \
        for (; tl + 3 * C_ < (TILES_); tl += 4 * C_) {                                            \
            const float4 v0 = sp[(size_t)tl * 8], v1 = sp[(size_t)(tl + C_) * 8];                 \
            const float4 v2 = sp[(size_t)(tl + 2 * C_) * 8], v3 = sp[(size_t)(tl + 3 * C_) * 8];  \
            ss_sum.x += (v0.x + v1.x) + (v2.x + v3.x);                                            \
            ss_sum.y += (v0.y + v1.y) + (v2.y + v3.y);                                            \
            ss_sum.z += (v0.z + v1.z) + (v2.z + v3.z);                                            \
            ss_sum.w += (v0.w + v1.w) + (v2.w + v3.w);                                            \
        }                                                                                         \
        for (; tl < (TILES_); tl += C_) {                                                         \
            const float4 v0 = sp[(size_t)tl * 8];                                                 \
            ss_sum.x += v0.x; ss_sum.y += v0.y; ss_sum.z += v0.z; ss_sum.w += v0.w;               \
        }                                                                                         \
    }
#define SK_SCALE_PUT(SS_)                                                                         \
    if ((SS_) != nullptr) {                                                                       \
        constexpr int Q_ = 4 * MG;                                                                \
        _Pragma("unroll") for (int o = Q_; o < 64; o <<= 1) {                                     \
            ss_sum.x += __shfl_xor(ss_sum.x, o, 64);                                              \
            ss_sum.y += __shfl_xor(ss_sum.y, o, 64);                                              \
            ss_sum.z += __shfl_xor(ss_sum.z, o, 64);                                              \
            ss_sum.w += __shfl_xor(ss_sum.w, o, 64);                                              \
        }                                                                                         \
        if ((threadIdx.x & 63) < Q_) *reinterpret_cast<float4*>(&ssr[threadIdx.x >> 6][(threadIdx.x % Q_) * 4]) = ss_sum; \
    }
#define SK_SCALE_GET(RSTD_, SS_, EPS_, WIDTH_, ROW_)                                              \
    if ((SS_) != nullptr) {                                                                       \
        float tot = 0.f;                                                                          \
        _Pragma("unroll") for (int c = 0; c < WAVES; ++c) tot += ssr[c][ROW_];                    \
        RSTD_ = 1.0f / sqrtf(tot / (float)(WIDTH_) + (EPS_));                                     \
    }

// The fused gate/up projection of a feed-forward with the SwiGLU in its epilogue (few rows of X):
// W holds the gate rows [0, I) and the up rows [I, 2I).  A tile of 16 W rows is the gate rows and the
// up rows of the same 8 outputs, so the thread that reduces gate (m, n) also reduces up (m, n) and
// stores act[m, n] = silu(gate) * up.  The intermediate [M, 2I] never goes to memory and the
// following projection reads plain rows.  Gate and up are rounded to bfloat16 before the
// activation, as the unfused path stores them.
template <int WAVES, int KSTEPS, int MG>
__global__ void __launch_bounds__(WAVES * 64)
gemm_gateup_swiglu_kernel(bf16* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W,
                          const bf16* __restrict__ bias, int M, int I, int K, int lda, int ldw, int ldc, int ntiles,
                          int ks, const float* __restrict__ SS, int ss_tiles, float eps) {
    // SS != null: X is r * w of a norm whose division is still to come (see SK_ROW_SCALE)
    static_assert(WAVES * 64 >= 128 * MG, "one reducing thread an output");
    __shared__ float part[2][MG][WAVES][64][4];
    __shared__ __attribute__((aligned(16))) float ssr[WAVES][32];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int s0 = wave * ks;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (K >> 3) - 1;
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
            xf[g][u] = (kok[u] && row < M) ? v : zero;
        }
    }
    // this lane's W row of tile t: rows 0..7 of the tile are gate rows 8 t .. 8 t + 7, rows 8..15 the up rows
    auto w_row = [&](int t) -> const uint4* {
        const int n = (t * 8 + (r & 7) < I) ? t * 8 + (r & 7) : I - 1;
        return reinterpret_cast<const uint4*>(W + (size_t)(n + (r >> 3) * I) * ldw);
    };
    uint4 a[KSTEPS];
    int tile = blockIdx.x;
    if (tile < ntiles) {
        const uint4* wp = w_row(tile);
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
    }
    // the reducing thread's output: row m, output j of the tile's 8
    const int et = threadIdx.x < 128 * MG ? threadIdx.x : 0;
    const int eg = et >> 7, m = eg * 16 + (et & 15), j = (et & 127) >> 4;
    const int gl = (j >> 2) * 16 + (et & 15), ge = j & 3;   // lane and element of the gate sum; up: lane + 32
    SK_SCALE_LOAD(SS, ss_tiles)
    float rstd = 1.0f;
    bool first = true;
    int buf = 0;
    for (; tile < ntiles; tile += gridDim.x) {
        f32x4 acc[MG];
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u)
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[g] = mfma16(a[u], xf[g][u], acc[g]);
        // the next tile's rows are on their way while this one is reduced
        const int next = tile + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        if (next < ntiles) {
            const uint4* wp = w_row(next);
#pragma unroll
            for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[buf][g][wave][lane][0]) = acc[g];
        if (first) SK_SCALE_PUT(SS)
        __syncthreads();
        if (first) SK_SCALE_GET(rstd, SS, eps, K, m < 32 ? m : 0)
        first = false;
        const int n = tile * 8 + j;
        if (threadIdx.x < 128 * MG && n < I && m < M) {
            float vg = 0.f, vu = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                vg += part[buf][eg][w][gl][ge];
                vu += part[buf][eg][w][gl + 32][ge];
            }
            vg *= rstd;
            vu *= rstd;
            if (bias != nullptr) {
                vg += to_f32(bias[n]);
                vu += to_f32(bias[n + I]);
            }
            vg = to_f32(from_f32<bf16>(vg));
            vu = to_f32(from_f32<bf16>(vu));
            C[(size_t)m * ldc + n] = from_f32<bf16>(vg / (1.0f + expf(-vg)) * vu);
        }
        buf ^= 1;  // the other buffer is free: its readers passed the barrier above one tile ago
    }
}

// The same with whole tiles: a workgroup multiplies the gate tile and the up tile of the same 16
// outputs one after the other (16 consecutive W rows a tile: 50.5 -> 47.0 us at the 8B shape), and the
// thread that reduces output (m, n) of the first also reduces (m, n) of the second.  For many tiles a
// workgroup; with few, the units of two tiles leave compute units idle at the end.
template <int WAVES, int KSTEPS, int MG>
__global__ void __launch_bounds__(WAVES * 64)
gemm_gateup_swiglu_pair_kernel(bf16* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W,
                          const bf16* __restrict__ bias, int M, int I, int K, int lda, int ldw, int ldc, int ntiles,
                          int ks, const float* __restrict__ SS, int ss_tiles, float eps) {
    static_assert(WAVES * 64 >= 256 * MG, "one reducing thread an output");
    __shared__ float part[2][MG][WAVES][64][4];
    __shared__ __attribute__((aligned(16))) float ssr[WAVES][32];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int s0 = wave * ks;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (K >> 3) - 1;
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
            xf[g][u] = (kok[u] && row < M) ? v : zero;
        }
    }
    // this lane's W row of a tile's gate half (0) or up half (1)
    auto w_row = [&](int t, int hf) -> const uint4* {
        const int n = (t * 16 + r < I) ? t * 16 + r : I - 1;
        return reinterpret_cast<const uint4*>(W + (size_t)(n + hf * I) * ldw);
    };
    uint4 a[KSTEPS];
    int tile = blockIdx.x;
    if (tile < ntiles) {
        const uint4* wp = w_row(tile, 0);
#pragma unroll
        for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
    }
    const int et = threadIdx.x < 256 * MG ? threadIdx.x : 0;
    const int eg = et >> 8, e = et & 3, l = (et & 255) >> 2;
    const int m = eg * 16 + (l & 15);
    SK_SCALE_LOAD(SS, ss_tiles)
    float rstd = 1.0f;
    bool first = true;
    int buf = 0;
    for (; tile < ntiles; tile += gridDim.x) {
        const int n = tile * 16 + (l >> 4) * 4 + e;
        const bool writer = threadIdx.x < 256 * MG && n < I && m < M;
        float val[2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            f32x4 acc[MG];
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < KSTEPS; ++u)
#pragma unroll
                for (int g = 0; g < MG; ++g) acc[g] = mfma16(a[u], xf[g][u], acc[g]);
            // the next tile's rows are on their way while this one is reduced
            const int nt = hf == 0 ? tile : tile + gridDim.x;
            __builtin_amdgcn_sched_barrier(0);
            if (nt < ntiles) {
                const uint4* wp = w_row(nt, hf == 0 ? 1 : 0);
#pragma unroll
                for (int u = 0; u < KSTEPS; ++u) a[u] = wp[k8c[u]];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[buf][g][wave][lane][0]) = acc[g];
            if (first) SK_SCALE_PUT(SS)
            __syncthreads();
            if (first) SK_SCALE_GET(rstd, SS, eps, K, m < 32 ? m : 0)
            first = false;
            float v = 0.f;
            if (threadIdx.x < 256 * MG) {
#pragma unroll
                for (int w = 0; w < WAVES; ++w) v += part[buf][eg][w][l][e];
                v *= rstd;
                if (bias != nullptr && writer) v += to_f32(bias[n + hf * I]);
            }
            val[hf] = to_f32(from_f32<bf16>(v));
            buf ^= 1;  // the other buffer is free: its readers passed the barrier above one tile ago
        }
        if (writer) C[(size_t)m * ldc + n] = from_f32<bf16>(val[0] / (1.0f + expf(-val[0])) * val[1]);
    }
}

// variant: 0 = choose; 4 = resident; 1, 2, 3, 5, 6 = shapes of the stream kernel (see below)
extern "C" int ilm_gemm_skinny(void* C, const void* X, const void* W, const void* bias, int M, int N,
                               int K, int lda, int ldw, int ldc, float alpha, int out_dtype, int variant,
                               hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: needs 1 <= M <= 64, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_skinny: K=%d lda=%d ldw=%d must be multiples of 8",
                K, lda, ldw);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_skinny: operands must be 16-byte aligned");
    ILM_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_skinny: strides too small");
    ILM_REQUIRE(out_dtype == ILM_DTYPE_BF16 || out_dtype == ILM_DTYPE_F32, "gemm_skinny: unknown output dtype %d", out_dtype);
    const int mg = (M + 15) / 16;
    const int ksteps = (K + 31) / 32;
    // two groups of 16 rows take the 8-wave shapes (256 registers a wave): K up to 8 * 16 k-steps
    const bool can_resident = (M <= 16 && ksteps <= 16 * 16) || (M <= 32 && ksteps <= 8 * 16);
    // measured on MI355X at the 8B shapes: resident wins where it applies, the 16-wave stream shape
    // for long K, two row tiles when X has more than 32 rows and W is tall
    if (variant == 0) variant = can_resident ? 4 : (M <= 16 ? 3 : (N >= 8192 ? 2 : 1));
    if (variant == 4) {
        ILM_REQUIRE(can_resident, "gemm_skinny: the resident kernel needs M <= 16 and K <= 8192, or M <= 32 and K <= 4096");
        const int ntiles = (N + 15) / 16;
#define SR_CASE(WV, KS, MGR, PER_CU, TC)                                                                    \
    {                                                                                                       \
        const int grid = ntiles < ilm_num_cus() * PER_CU ? ntiles : ilm_num_cus() * PER_CU;                         \
        gemm_skinny_resident_kernel<WV, KS, MGR, TC><<<grid, WV * 64, 0, stream>>>(                         \
            (TC*)C, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, N, K, lda, ldw, ldc, alpha, ntiles, \
            (ksteps + WV - 1) / WV);                                                                        \
    }
        // measured on MI355X at K = 4096: 8 waves of 16 k-steps (more loads in flight a wave) win where the
        // tiles are at most one a compute unit (o projection, 9.1 against 10.2 us) or many (gate/up 47.8
        // against 50.0 us, the head), 16 waves of 8 where they are a few more than the compute units
        // (q/k/v).  Two tiles in flight instead of one changed nothing.  INFINILM_AMD_SKINNY_FAT=0: always 16 x 8.
        static int fat = -1;
        if (fat < 0) { const char* e = getenv("INFINILM_AMD_SKINNY_FAT"); fat = e ? atoi(e) : 1; }
        const bool fat_waves = fat && ksteps > 8 * 8 && ksteps <= 8 * 16 && (ntiles <= ilm_num_cus() || ntiles >= 4 * ilm_num_cus());
#define SR_DISPATCH(TC)                                         \
    if (mg == 2) {                                              \
        if (ksteps <= 8 * 4) SR_CASE(8, 4, 2, 2, TC)            \
        else if (ksteps <= 8 * 8) SR_CASE(8, 8, 2, 2, TC)       \
        else if (ksteps <= 8 * 12) SR_CASE(8, 12, 2, 1, TC)     \
        else SR_CASE(8, 16, 2, 1, TC)                           \
    }                                                           \
    else if (ksteps <= 8 * 4) SR_CASE(8, 4, 1, 2, TC)           \
    else if (ksteps <= 8 * 8) SR_CASE(8, 8, 1, 2, TC)           \
    else if (fat_waves && ksteps <= 8 * 12) SR_CASE(8, 12, 1, 2, TC) \
    else if (fat_waves) SR_CASE(8, 16, 1, 2, TC)                \
    else if (ksteps <= 16 * 8) SR_CASE(16, 8, 1, 1, TC)         \
    else if (ksteps <= 16 * 12) SR_CASE(16, 12, 1, 1, TC)       \
    else SR_CASE(16, 16, 1, 1, TC)
        if (out_dtype == ILM_DTYPE_BF16) { SR_DISPATCH(bf16) } else { SR_DISPATCH(float) }
#undef SR_DISPATCH
#undef SR_CASE
        ILM_LAUNCH_CHECK("gemm_skinny_resident");
        return 0;
    }
    // variants of the stream kernel: (waves, row tiles, unroll)
    int wv = 8, rt = 1, unroll = 4;
    if (variant == 2) rt = 2;
    else if (variant == 3) { wv = 16; unroll = 2; }
    else if (variant == 5) { wv = 16; rt = 2; unroll = 2; }
    else if (variant == 6) { wv = 16; unroll = 4; }
    else ILM_REQUIRE(variant == 1, "gemm_skinny: unknown variant %d", variant);
    if (mg > 2 && wv == 16 && rt == 2) wv = 8;  // LDS for the partial tiles
    const int grid = (N + 16 * rt - 1) / (16 * rt);
#define SK_CASE(WV, MG, RT, U, TC)                                                                          \
    gemm_skinny_stream_kernel<WV, MG, RT, U, TC><<<grid, WV * 64, 0, stream>>>(                             \
        (TC*)C, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, N, K, lda, ldw, ldc, alpha)
#define SK_MG(WV, RT, U, TC)                    \
    switch (mg) {                               \
        case 1: SK_CASE(WV, 1, RT, U, TC); break; \
        case 2: SK_CASE(WV, 2, RT, U, TC); break; \
        case 3: SK_CASE(WV, 3, RT, U, TC); break; \
        default: SK_CASE(WV, 4, RT, U, TC); break; \
    }
#define SK_SHAPE(TC)                                              \
    if (wv == 8 && rt == 1) { SK_MG(8, 1, 4, TC) }                \
    else if (wv == 8 && rt == 2) { SK_MG(8, 2, 4, TC) }           \
    else if (wv == 16 && rt == 1 && unroll == 2) { SK_MG(16, 1, 2, TC) } \
    else if (wv == 16 && rt == 1) { SK_MG(16, 1, 4, TC) }         \
    else if (mg == 1) { SK_CASE(16, 1, 2, 2, TC); }               \
    else { SK_CASE(16, 2, 2, 2, TC); }
    if (out_dtype == ILM_DTYPE_BF16) { SK_SHAPE(bf16) } else { SK_SHAPE(float) }
#undef SK_SHAPE
#undef SK_MG
#undef SK_CASE
    ILM_LAUNCH_CHECK("gemm_skinny_stream");
    return 0;
}

// act [M, ldc] = silu(X Wg^T + bg) * (X Wu^T + bu) with W = [Wg; Wu] of 2 I rows (bias of 2 I entries or null).
// ss != null: X is r * w of the RMS norm before the projection, not yet divided by the rows' root mean square, and
// ss [ss_tiles][32] holds partial sums of squares of the rows of r (what ilm_gemm_tail leaves): the kernel adds them
// up and applies 1 / sqrt(sum / K + eps) to its sums (K is also the norm's width).
extern "C" int ilm_gemm_gateup_swiglu(void* C, int ldc, const void* X, int lda, const void* W, int ldw, const void* bias,
                                      int M, int I, int K, const void* ss, int ss_tiles, float eps, hipStream_t stream) {
    ILM_REQUIRE(ss == nullptr || ss_tiles > 0, "gemm_gateup_swiglu: no tiles of partial sums");
    ILM_REQUIRE(M > 0 && M <= 32 && I > 0 && K > 0, "gemm_gateup_swiglu: needs 1 <= M <= 32, got M=%d I=%d K=%d", M, I, K);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldc >= I,
                "gemm_gateup_swiglu: K=%d lda=%d ldw=%d ldc=%d", K, lda, ldw, ldc);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_gateup_swiglu: operands must be 16-byte aligned");
    const int ksteps = (K + 31) / 32;
    ILM_REQUIRE(ksteps <= (M <= 16 ? 16 * 16 : 8 * 16), "gemm_gateup_swiglu: K=%d is beyond %d", K, M <= 16 ? 8192 : 4096);
    // whole tiles in pairs where every workgroup gets at least two pairs, else tiles of 8 + 8 rows
    const bool pairs = (I + 15) / 16 >= 2 * ilm_num_cus();
    const int ntiles = pairs ? (I + 15) / 16 : (I + 7) / 8;
#define GU_LAUNCH(KERNEL, WV, KS, MGR, PER_CU)                                                              \
    {                                                                                                       \
        const int grid = ntiles < ilm_num_cus() * PER_CU ? ntiles : ilm_num_cus() * PER_CU;                         \
        KERNEL<WV, KS, MGR><<<grid, WV * 64, 0, stream>>>(                                                  \
            (bf16*)C, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, I, K, lda, ldw, ldc, ntiles,    \
            (ksteps + WV - 1) / WV, (const float*)ss, ss_tiles, eps);                                       \
    }
#define GU_CASE(WV, KS, MGR, PER_CU)                                                       \
    {                                                                                      \
        if (pairs) GU_LAUNCH(gemm_gateup_swiglu_pair_kernel, WV, KS, MGR, PER_CU)          \
        else GU_LAUNCH(gemm_gateup_swiglu_kernel, WV, KS, MGR, PER_CU)                     \
    }
    if (M > 16) {
        if (ksteps <= 8 * 4) GU_CASE(8, 4, 2, 2)
        else if (ksteps <= 8 * 8) GU_CASE(8, 8, 2, 2)
        else if (ksteps <= 8 * 12) GU_CASE(8, 12, 2, 1)
        else GU_CASE(8, 16, 2, 1)
    }
    else if (ksteps <= 8 * 4) GU_CASE(8, 4, 1, 2)
    else if (ksteps <= 8 * 8) GU_CASE(8, 8, 1, 2)
    else if (ksteps <= 8 * 12) GU_CASE(8, 12, 1, 2)   // (a width like 2304: 9 of 12 slots a wave instead of 9 of 16)
    else if (ksteps <= 8 * 16) GU_CASE(8, 16, 1, 2)
    else if (ksteps <= 16 * 12) GU_CASE(16, 12, 1, 1)
    else GU_CASE(16, 16, 1, 1)
#undef GU_LAUNCH
#undef GU_CASE
    ILM_LAUNCH_CHECK("gemm_gateup_swiglu");
    return 0;
}
