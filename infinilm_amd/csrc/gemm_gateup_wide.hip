// The fused gate/up projection of a feed-forward with the SwiGLU in its epilogue for 33 to 64 rows
// of X (bfloat16): act[M, I] = silu(X Wg^T + bg) * (X Wu^T + bu), W = [Wg; Wu].  A decode step with
// many requests: bound by reading W once, but with too many rows for the X fragments of a whole K
// to stay in registers.
//
// A workgroup of 8 waves takes 64 outputs; a wave takes 8 of them: its 16-row tile of W is the 8
// gate rows and the 8 up rows of the same outputs, streamed over the whole K straight into
// v_mfma_f32_16x16x32_bf16 fragments, one step of 256 ahead: a step's loads of a wave take 512 bytes
// of each of its 16 rows (steps of 128, 256 bytes a row at a time, reached 3.7 TB/s at the 8B shape
// however many were in flight; steps of 256 reach 4.3; two or three steps ahead instead of one
// lose again).  The X tile of a step is staged in LDS (double-buffered, one barrier a step) and
// shared by the waves.  No reduction between waves: a
// wave owns its outputs, and a lane with gate sums gets the up sums of the same outputs from the
// lane 32 further on, rounds both to bfloat16 (as the unfused path stores them) and stores
// silu(gate) * up.  The [M, 2I] intermediate never goes to memory.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define GW_WAVES 8
#define GW_THREADS (GW_WAVES * 64)
#define GW_KT 256                 // k per step
#define GW_KSUB (GW_KT / 32)      // matrix-core k-steps a step
#define GW_NOUT (GW_WAVES * 8)    // outputs a workgroup
#define GW_AHEAD 1                // steps the W fragments are loaded ahead

__device__ __forceinline__ f32x4 gw_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// MG: groups of 16 rows of X (2 to 4).  FRAGW: W is given in fragment order (frag.h), tiles of 8 gate rows and the 8
// up rows of the same outputs: a wave's W fragment is then 1 KB of consecutive bytes.
template <int MG, bool FRAGW>
__global__ void __launch_bounds__(GW_THREADS)
gemm_gateup_wide_kernel(bf16* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W,
                        const bf16* __restrict__ bias, int M, int I, int K, int lda, int ldw, int ldc) {
    constexpr int MP = MG * 16;
    constexpr int XROW = GW_KT + 8;                       // padded LDS row: 16 rows x 16 bytes fall on distinct banks
    constexpr int PR = GW_KT / 8;                         // 16-byte pieces of a row of an X tile
    constexpr int RPP = GW_THREADS / PR;                  // rows the threads cover at once
    constexpr int XPER = MP / RPP;                        // pieces a thread: rows tid / PR + RPP i
    static_assert(MP % RPP == 0 && XPER <= 8, "an X tile is at most eight 16-byte pieces a thread");
    __shared__ __attribute__((aligned(16))) bf16 Xs[2][MP][XROW];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
    const int n0 = (blockIdx.x * GW_WAVES + wave) * 8;    // this wave's first output
    const int nsteps = (K + GW_KT - 1) / GW_KT;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int k8_last = (K >> 3) - 1;

    // this lane's W row: rows 0..7 of the tile are gate rows, rows 8..15 the up rows of the same outputs
    // (clamped; outputs beyond I are never stored)
    const int nr = (n0 + (r & 7) < I) ? n0 + (r & 7) : I - 1;
    const int ksteps = (K + 31) >> 5;
    const uint4* wp = FRAGW ? reinterpret_cast<const uint4*>(W) + (size_t)(blockIdx.x * GW_WAVES + wave) * ksteps * 64 + lane
                            : reinterpret_cast<const uint4*>(W + (size_t)(nr + (r >> 3) * I) * ldw);
    // this thread's pieces of an X tile: k offset (tid % PR) * 8 of rows tid / PR + RPP i
    const int xk = threadIdx.x % PR, xr = threadIdx.x / PR;
    bf16* xs = &Xs[0][xr][xk * 8];
    constexpr int XBUF = MP * XROW;   // elements between the two buffers

    // Loads are unconditional 16-byte loads from clamped addresses; what lies beyond K or beyond M is
    // replaced by zeros on the X side, which makes the clamped W loads harmless.  The X pieces are plain
    // variables: a register array indexed inside a macro's loop lands in scratch memory, and every
    // access to that waits for all loads in flight.  A piece is looked at only when it is stored into LDS (a
    // select right after its load would make the wave wait for it there), and the next step's loads are issued
    // without a branch around them (after the last step: that step's again, for nothing): behind a branch the
    // compiler cannot count how many loads are younger than the fragments it is about to use, and waits for the
    // new ones.
#define GW_LOAD_W(DST_, STEP_)                                                   \
    _Pragma("unroll") for (int s = 0; s < GW_KSUB; ++s) {                        \
        if (FRAGW) {                                                             \
            const int st = (STEP_) * GW_KSUB + s;                                \
            DST_[s] = wp[(size_t)(st < ksteps ? st : ksteps - 1) * 64];          \
        } else {                                                                 \
            const int k8 = (STEP_) * PR + s * 4 + q;                             \
            DST_[s] = wp[k8 <= k8_last ? k8 : k8_last];                          \
        }                                                                        \
    }
#define GW_X1(XV_, I_)                                                           \
    if (XPER > I_) {                                                             \
        const int row = xr + RPP * I_;                                           \
        XV_ = *reinterpret_cast<const uint4*>(X + (size_t)(row < M ? row : 0) * lda + (size_t)k8c * 8); \
    }
#define GW_LOAD_X(STEP_)                                                         \
    {                                                                            \
        const int k8 = (STEP_) * PR + xk;                                        \
        const int k8c = k8 <= k8_last ? k8 : k8_last;                            \
        GW_X1(x0, 0) GW_X1(x1, 1) GW_X1(x2, 2) GW_X1(x3, 3) GW_X1(x4, 4) GW_X1(x5, 5) GW_X1(x6, 6) GW_X1(x7, 7) \
    }
#define GW_S1(XV_, I_, B_)                                                                           \
    if (XPER > I_) {                                                                                 \
        const unsigned mk = (kin && xr + RPP * I_ < M) ? 0xffffffffu : 0u;   /* (a select between two 16-byte structs goes through memory) */ \
        *reinterpret_cast<uint4*>(xs + (B_) * XBUF + RPP * I_ * XROW) = make_uint4(XV_.x & mk, XV_.y & mk, XV_.z & mk, XV_.w & mk); \
    }
#define GW_STORE_X(BUF_, STEP_)                                                  \
    {                                                                            \
        const bool kin = (STEP_) * PR + xk <= k8_last;                           \
        GW_S1(x0, 0, BUF_) GW_S1(x1, 1, BUF_) GW_S1(x2, 2, BUF_) GW_S1(x3, 3, BUF_) GW_S1(x4, 4, BUF_) GW_S1(x5, 5, BUF_) GW_S1(x6, 6, BUF_) GW_S1(x7, 7, BUF_) \
    }

    f32x4 acc[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
    uint4 x0 = zero, x1 = zero, x2 = zero, x3 = zero, x4 = zero, x5 = zero, x6 = zero, x7 = zero;
    // W fragments of GW_AHEAD + 1 steps in turn; the loop below is unrolled over the sets, so every index is a constant
    uint4 w[GW_AHEAD + 1][GW_KSUB];
    GW_LOAD_X(0)
#pragma unroll
    for (int j = 0; j < GW_AHEAD; ++j)
        if (j < nsteps) GW_LOAD_W(w[j], j)
    GW_STORE_X(0, 0)
    __syncthreads();
    for (int base = 0; base < nsteps; base += GW_AHEAD + 1) {
#pragma unroll
        for (int j = 0; j <= GW_AHEAD; ++j) {
            const int step = base + j;
            if (step < nsteps) {   // uniform over the workgroup
                const int buf = step & 1;
                // X of the next step first: the wait for it before the store below then leaves the W loads,
                // issued later and coming from memory, in flight
                {
                    const int nx = step + 1 < nsteps ? step + 1 : nsteps - 1;
                    const int nw = step + GW_AHEAD < nsteps ? step + GW_AHEAD : nsteps - 1;
                    GW_LOAD_X(nx)
                    GW_LOAD_W(w[(j + GW_AHEAD) % (GW_AHEAD + 1)], nw)
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < GW_KSUB; ++s) {
                    uint4 b[MG];
#pragma unroll
                    for (int g = 0; g < MG; ++g)
                        b[g] = *reinterpret_cast<const uint4*>(&Xs[buf][g * 16 + r][s * 32 + q * 8]);
#pragma unroll
                    for (int g = 0; g < MG; ++g) acc[g] = gw_mfma(w[j][s], b[g], acc[g]);
                }
                __builtin_amdgcn_sched_barrier(0);
                // (its readers passed the barrier one step ago; after the last step the stored tile is not read: the
                // store is unconditional so that the compiler does not move the loads down into a branch beside it)
                GW_STORE_X(buf ^ 1, step + 1 < nsteps ? step + 1 : nsteps - 1)
                __syncthreads();
            }
        }
    }
#undef GW_LOAD_W
#undef GW_LOAD_X
#undef GW_X1
#undef GW_S1
#undef GW_STORE_X
    // acc[g][e] of lane (r, q): token g*16 + r, tile row q*4 + e: gate rows for q < 2, up rows for q >= 2.
    // The lane 32 further on holds the up sums of this lane's outputs.
    const int n = n0 + q * 4;
    float bg[4] = {0.f, 0.f, 0.f, 0.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias != nullptr && q < 2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int ne = n + e < I ? n + e : I - 1;
            bg[e] = to_f32(bias[ne]);
            bu[e] = to_f32(bias[ne + I]);
        }
    }
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        float up[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) up[e] = __shfl_xor(acc[g][e], 32, 64);
        const int m = g * 16 + r;
        if (q >= 2 || m >= M) continue;
        bf16 o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float vg = to_f32(from_f32<bf16>(acc[g][e] + bg[e]));
            const float vu = to_f32(from_f32<bf16>(up[e] + bu[e]));
            o[e] = from_f32<bf16>(vg / (1.0f + expf(-vg)) * vu);
        }
        bf16* dst = C + (size_t)m * ldc + n;
        if (n + 3 < I && (ldc & 3) == 0 && ((uintptr_t)C & 7) == 0) {
            *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(o);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < I) dst[e] = o[e];
        }
    }
}

// act [M, ldc] = silu(X Wg^T + bg) * (X Wu^T + bu) with W = [Wg; Wu] of 2 I rows (bias of 2 I entries or null),
// 17 <= M <= 64 (made for 33 to 64: below, the kernels that keep X in registers are faster).
// frag_w != 0: W is the weight in fragment order with tiles of 8 gate + 8 up rows (ldw is not used).
extern "C" int ilm_gemm_gateup_wide(void* C, int ldc, const void* X, int lda, const void* W, int ldw, const void* bias,
                                    int M, int I, int K, int frag_w, hipStream_t stream) {
    ILM_REQUIRE(M > 16 && M <= 64 && I > 0 && K > 0, "gemm_gateup_wide: needs 17 <= M <= 64, got M=%d I=%d K=%d", M, I, K);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && (frag_w || (ldw % 8 == 0 && ldw >= K)) && lda >= K && ldc >= I,
                "gemm_gateup_wide: K=%d lda=%d ldw=%d ldc=%d", K, lda, ldw, ldc);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_gateup_wide: operands must be 16-byte aligned");
    const int grid = (I + GW_NOUT - 1) / GW_NOUT;
    const bf16* b = (const bf16*)bias;
#define GW_GO(MG_)                                                                                                          \
    if (frag_w) gemm_gateup_wide_kernel<MG_, true><<<grid, GW_THREADS, 0, stream>>>((bf16*)C, (const bf16*)X, (const bf16*)W, b, M, I, K, lda, ldw, ldc); \
    else gemm_gateup_wide_kernel<MG_, false><<<grid, GW_THREADS, 0, stream>>>((bf16*)C, (const bf16*)X, (const bf16*)W, b, M, I, K, lda, ldw, ldc);
    if (M <= 32) { GW_GO(2) } else if (M <= 48) { GW_GO(3) } else { GW_GO(4) }
#undef GW_GO
    ILM_LAUNCH_CHECK("gemm_gateup_wide");
    return 0;
}
