// Products with 17 to 208 rows of X (bfloat16) whose result goes into the residual sum: o and down
// projections of a decode step with many requests, or of a small portion of a prompt.  There the
// vendor library leaves most of the chip idle (few output tiles, long K); here K is split over
// blockIdx.y into float partial results C[y][M][N] that the next add+RMSNorm sums in order, so
// that a product of 4096 columns still makes 512 workgroups.
//
// A workgroup of 8 waves takes 128 rows of W (16 a wave) and one K range, in steps of 128 (64 above
// 64 rows of X): the X tile of a step is staged in LDS (double-buffered, one barrier a step) and
// shared by the waves; each wave streams its own W rows straight into v_mfma_f32_16x16x32_bf16
// fragments, one step ahead.  A step moves 32 KB of W: with memory latencies of a microsecond or
// two, steps have to be this large for two workgroups a compute unit to keep the memory busy.
// No reduction between waves.  ACT: X holds rows [gate | up] of 2K elements and the tile is
// made on the way into LDS, x = silu(gate) * up (the SwiGLU between the two projections of a
// feed-forward): no activation tensor in memory.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

#define GM_WAVES 8
#define GM_NT (GM_WAVES * 16)   // W rows a workgroup
#define GM_THREADS (GM_WAVES * 64)

__device__ __forceinline__ f32x4 gm_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ uint4 gm_swiglu8(uint4 g, uint4 up) {
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {up.x, up.y, up.z, up.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
        // hardware exp2 and reciprocal (about 1 ulp each): the result is rounded to bfloat16 anyway
        const float s0 = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g0));
        const float s1 = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g1));
        const f32x2 pr = {g0 * s0 * u0, g1 * s1 * u1};
        o[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2));
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// MG: groups of 16 rows of X (2 .. 13); KT: k per step (128, or 64 where the X tiles would not fit)
template <int MG, int KT, bool ACT>
__global__ void __launch_bounds__(GM_THREADS, 4)
gemm_mid_kernel(float* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W, int M, int N, int K,
                int lda, int ldw, int ldc, int kspan, size_t c_part_stride) {
    constexpr int MP = MG * 16;
    constexpr int KSUB = KT / 32;                       // matrix-core k-steps a step
    constexpr int XROW = KT + 8;                        // padded LDS row: 16 rows x 16 bytes fall on distinct banks
    constexpr int XPIECES = MP * (KT / 8);              // 16-byte pieces of an X tile
    constexpr int XPER = (XPIECES + GM_THREADS - 1) / GM_THREADS;
    __shared__ __attribute__((aligned(16))) bf16 Xs[2][MP][XROW];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * GM_NT + wave * 16;
    const int k_lo = blockIdx.y * kspan;
    const int k_hi = (k_lo + kspan < K) ? k_lo + kspan : K;
    const int nsteps = (k_hi - k_lo + KT - 1) / KT;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (k_hi >> 3) - 1;   // last valid 16-byte piece of a row in this K range

    // this wave's W rows (clamped; the stores are masked)
    const int wrow = (n0 + r < N) ? n0 + r : N - 1;
    const uint4* wp = reinterpret_cast<const uint4*>(W + (size_t)wrow * ldw);
    // this thread's (at most two) pieces of an X tile: piece pc -> row pc / (KT/8), k offset (pc % (KT/8)) * 8.
    // Plain variables, not arrays: indexed arrays of registers end up in scratch memory here, and
    // every access to that waits for all loads in flight.
    static_assert(XPER <= 4, "an X tile is at most four 16-byte pieces a thread");
    static_assert(sizeof(bf16) * 2 * MP * XROW <= 65536, "the two X tiles fit the LDS of a workgroup");
    const int pc0 = threadIdx.x, pc1 = threadIdx.x + GM_THREADS, pc2 = threadIdx.x + 2 * GM_THREADS, pc3 = threadIdx.x + 3 * GM_THREADS;
    const int xk0 = pc0 % (KT / 8), xk1 = pc1 % (KT / 8), xk2 = pc2 % (KT / 8), xk3 = pc3 % (KT / 8);
    const bool xok0 = pc0 < XPIECES && pc0 / (KT / 8) < M, xok1 = XPER > 1 && pc1 < XPIECES && pc1 / (KT / 8) < M;
    const bool xok2 = XPER > 2 && pc2 < XPIECES && pc2 / (KT / 8) < M, xok3 = XPER > 3 && pc3 < XPIECES && pc3 / (KT / 8) < M;
    const uint4* xp0 = reinterpret_cast<const uint4*>(X + (size_t)(xok0 ? pc0 / (KT / 8) : 0) * lda);
    const uint4* xp1 = reinterpret_cast<const uint4*>(X + (size_t)(xok1 ? pc1 / (KT / 8) : 0) * lda);
    const uint4* xp2 = reinterpret_cast<const uint4*>(X + (size_t)(xok2 ? pc2 / (KT / 8) : 0) * lda);
    const uint4* xp3 = reinterpret_cast<const uint4*>(X + (size_t)(xok3 ? pc3 / (KT / 8) : 0) * lda);
    bf16* xs0 = &Xs[0][(pc0 < XPIECES ? pc0 : 0) / (KT / 8)][xk0 * 8];
    bf16* xs1 = &Xs[0][(pc1 < XPIECES ? pc1 : 0) / (KT / 8)][xk1 * 8];
    bf16* xs2 = &Xs[0][(pc2 < XPIECES ? pc2 : 0) / (KT / 8)][xk2 * 8];
    bf16* xs3 = &Xs[0][(pc3 < XPIECES ? pc3 : 0) / (KT / 8)][xk3 * 8];
    constexpr int XBUF = MP * XROW;   // elements between the two buffers
#define GM_X_PIECE(DST_, XP_, XK_, OK_, STEP_)                                                     \
    {                                                                                              \
        const int k8 = ((k_lo + (STEP_) * KT) >> 3) + XK_;                                         \
        const int k8c = k8 <= k8_last ? k8 : k8_last;                                              \
        uint4 v = XP_[k8c];                                                                        \
        if (ACT) v = gm_swiglu8(v, XP_[k8c + (K >> 3)]);                                           \
        /* zeros beyond M and beyond K make clamped W loads harmless */                            \
        DST_ = (OK_ && k8 <= k8_last) ? v : zero;                                                  \
    }
#define GM_LOAD_X(STEP_)                                                                           \
    GM_X_PIECE(x0, xp0, xk0, xok0, STEP_)                                                          \
    if (XPER > 1) GM_X_PIECE(x1, xp1, xk1, xok1, STEP_)                                            \
    if (XPER > 2) GM_X_PIECE(x2, xp2, xk2, xok2, STEP_)                                            \
    if (XPER > 3) GM_X_PIECE(x3, xp3, xk3, xok3, STEP_)
#define GM_STORE_X(BUF_)                                                                           \
    if (pc0 < XPIECES) *reinterpret_cast<uint4*>(xs0 + (BUF_) * XBUF) = x0;                        \
    if (XPER > 1 && pc1 < XPIECES) *reinterpret_cast<uint4*>(xs1 + (BUF_) * XBUF) = x1;        \
    if (XPER > 2 && pc2 < XPIECES) *reinterpret_cast<uint4*>(xs2 + (BUF_) * XBUF) = x2;        \
    if (XPER > 3 && pc3 < XPIECES) *reinterpret_cast<uint4*>(xs3 + (BUF_) * XBUF) = x3;
#define GM_LOAD_W(DST_, STEP_)                                                                     \
    _Pragma("unroll") for (int s = 0; s < KSUB; ++s) {                                             \
        const int k8 = ((k_lo + (STEP_) * KT) >> 3) + s * 4 + q;                                   \
        DST_[s] = wp[k8 <= k8_last ? k8 : k8_last];                                                \
    }

    f32x4 acc[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
    uint4 x0 = zero, x1 = zero, x2 = zero, x3 = zero, wa[KSUB], wb[KSUB];
    GM_LOAD_W(wa, 0)
    GM_LOAD_X(0)
    GM_STORE_X(0)
    __syncthreads();
    // two steps an iteration, so that the W fragments of the step in flight alternate between two sets
#define GM_STEP(WCUR_, WNEXT_, STEP_)                                                              \
    {                                                                                              \
        const int buf = (STEP_) & 1;                                                               \
        if ((STEP_) + 1 < nsteps) {                                                                \
            /* X first: the wait for it before the store below then leaves the W loads, issued   \
               later and coming from memory, in flight into the next step */                      \
            GM_LOAD_X((STEP_) + 1)                                                                 \
            GM_LOAD_W(WNEXT_, (STEP_) + 1)                                                         \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        _Pragma("unroll") for (int s = 0; s < KSUB; ++s) {                                         \
            uint4 b[MG];                                                                           \
            _Pragma("unroll") for (int g = 0; g < MG; ++g)                                         \
                b[g] = *reinterpret_cast<const uint4*>(&Xs[buf][g * 16 + r][s * 32 + q * 8]);      \
            _Pragma("unroll") for (int g = 0; g < MG; ++g) acc[g] = gm_mfma(WCUR_[s], b[g], acc[g]); \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        if ((STEP_) + 1 < nsteps) GM_STORE_X(buf ^ 1)   /* its readers passed the barrier one step ago */ \
        __syncthreads();                                                                           \
    }
    for (int step = 0; step < nsteps; step += 2) {
        GM_STEP(wa, wb, step)
        if (step + 1 < nsteps) GM_STEP(wb, wa, step + 1)
    }
#undef GM_STEP
#undef GM_LOAD_X
#undef GM_X_PIECE
#undef GM_STORE_X
#undef GM_LOAD_W
    // lane (r, q): X row g*16 + r, W rows n0 + q*4 + e
    float* Cp = C + (size_t)blockIdx.y * c_part_stride;
    const int n = n0 + q * 4;
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        const int m = g * 16 + r;
        if (m >= M) continue;
        float* dst = Cp + (size_t)m * ldc + n;
        if (n + 3 < N && (ldc & 3) == 0) {
            *reinterpret_cast<f32x4*>(dst) = acc[g];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < N) dst[e] = acc[g][e];
        }
    }
}

// C: float [kb][M][ldc] with c_part_stride elements between the parts; part y covers K range
// [y * kspan, (y + 1) * kspan), kspan a multiple of 128.  act != 0: X rows are [gate | up] (2K long).
extern "C" int ilm_gemm_mid(void* C, int ldc, long c_part_stride, int kb, int kspan, const void* W, int ldw, int M, int N,
                            int K, const void* X, int lda, int act, hipStream_t stream) {
    ILM_REQUIRE(M > 16 && M <= 208 && N > 0 && K > 0, "gemm_mid: needs 17 <= M <= 208, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 8 == 0 && ldw % 8 == 0 && lda % 8 == 0 && ldw >= K && ldc >= N && lda >= (act ? 2 * K : K),
                "gemm_mid: K=%d lda=%d ldw=%d ldc=%d", K, lda, ldw, ldc);
    ILM_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)C & 15) == 0 && (!act || K % 8 == 0),
                "gemm_mid: operands must be 16-byte aligned");
    ILM_REQUIRE(kb >= 1 && kb <= 65535 && kspan > 0 && kspan % 128 == 0 && (long)kb * kspan >= K &&
                    (long)(kb - 1) * kspan < K, "gemm_mid: %d parts of %d do not cover K=%d", kb, kspan, K);
    dim3 grid((N + GM_NT - 1) / GM_NT, kb);
#define GM_LAUNCH(MG_)                                                                                        \
    if (act) gemm_mid_kernel<MG_, (MG_ <= 4 ? 128 : 64), true><<<grid, GM_THREADS, 0, stream>>>(              \
        (float*)C, (const bf16*)X, (const bf16*)W, M, N, K, lda, ldw, ldc, kspan, (size_t)c_part_stride);     \
    else gemm_mid_kernel<MG_, (MG_ <= 4 ? 128 : 64), false><<<grid, GM_THREADS, 0, stream>>>(                 \
        (float*)C, (const bf16*)X, (const bf16*)W, M, N, K, lda, ldw, ldc, kspan, (size_t)c_part_stride)
    switch ((M + 15) / 16) {
        case 2: GM_LAUNCH(2); break;
        case 3: GM_LAUNCH(3); break;
        case 4: GM_LAUNCH(4); break;
        case 5: GM_LAUNCH(5); break;
        case 6: GM_LAUNCH(6); break;
        case 7: GM_LAUNCH(7); break;
        case 8: GM_LAUNCH(8); break;
        case 9: GM_LAUNCH(9); break;
        case 10: GM_LAUNCH(10); break;
        case 11: GM_LAUNCH(11); break;
        case 12: GM_LAUNCH(12); break;
        default: GM_LAUNCH(13); break;
    }
#undef GM_LAUNCH
    ILM_LAUNCH_CHECK("gemm_mid");
    return 0;
}
