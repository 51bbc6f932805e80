// Products of 17 to 208 rows of X (bfloat16) with W streamed once and long chunks of X resident in LDS: the
// projections of a decode step with many requests, or of a small portion of a prompt.
//
// A workgroup of 8 waves takes 128 rows of W (a tile of 16 a wave) and all rows of X, and walks its range of K in
// chunks of KC = 64 or 128 k, two of which lie in LDS.  A chunk of X goes from plain rows into LDS in fragment
// order: whole 128-byte lines of 8 rows an instruction on the memory side, and on the LDS side the 1 KB that one
// matrix operand reads lies in the lanes' order, so neither padding nor exchange of pieces is needed for reads
// without bank conflicts.  The next chunk's X (in registers) and W fragments are on their way while this one is
// multiplied, one barrier a chunk.  Up to 128 rows of X a workgroup stays within 128 registers and 64 KB of LDS,
// so that two share a compute unit and one's barrier and waits are covered by the other (measured at the 8B
// shapes: chunks of 256 and 512 k, which fill the unit's 160 KB of LDS with one workgroup, were slower at every
// row count: gate/up at 64 rows 56.2 and 58.3 us against 53.2 with chunks of 128).  A wave streams its
// own W rows straight into v_mfma_f32_16x16x32_bf16 fragments (from plain rows, or 1 KB of consecutive bytes a
// fragment where the weight is given in fragment order, frag.h); no reduction between waves.
//
//   parts    C[y][M][N] float: K split over blockIdx.y, summed in order by the next add+RMSNorm (o and down
//            projections: few output tiles and a long K)
//   swiglu   a tile is the 8 gate rows and the 8 up rows of the same outputs: act = silu(gate) * up in
//            bfloat16 rows, gate and up rounded to bfloat16 first, as the unfused path stores them
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define GT_WAVES 8
#define GT_THREADS (GT_WAVES * 64)
#define GT_NT (GT_WAVES * 16)   // W rows a workgroup

enum { GT_PARTS = 0, GT_SWIGLU = 1 };

struct GtArgs {
    const bf16* X;
    const bf16* W;
    const bf16* bias;   // swiglu: [2 I] or null
    int M, N, K;        // N: rows of W (parts), outputs I (swiglu: W has 2 I rows)
    int lda, ldw;
    int chunks, chunks_per_part;
    float* C;           // parts
    int ldc;
    size_t part_stride;
    bf16* act;          // swiglu
    int ld_act;
};

__device__ __forceinline__ f32x4 gt_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// MG: groups of 16 rows of X; KC: k a chunk; FRAGW: W in fragment order (parts: tiles of 16 consecutive rows; swiglu:
// tiles of 8 gate + 8 up rows)
template <int MG, int KC, bool FRAGW, int EPI>
__global__ void __launch_bounds__(GT_THREADS, MG <= 8 ? 4 : 2)
gemm_tall_kernel(const GtArgs A) {
    constexpr int KS = KC / 32;                 // matrix-core k-steps a chunk
    constexpr int LINES = KC / 64;              // 128-byte lines a row of a chunk
    constexpr int BLOCKS = MG * 2 * LINES;      // staging blocks (8 rows x one line) a chunk
    constexpr int XPER = (BLOCKS + GT_WAVES - 1) / GT_WAVES;
    static_assert(XPER <= 8, "a chunk of X is at most eight 16-byte pieces a thread");
    static_assert(KC == 64 || KC == 128, "chunks of 64 or 128 k");
    static_assert(2 * KS * MG <= (MG <= 8 ? 64 : 144), "two chunks of X fit the LDS (of half a compute unit up to 128 rows)");
    __shared__ __align__(16) uint4 Xs[2][KS][MG][64];
    // the wave's number as a scalar: what depends on it stays in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int r8 = lane & 7, pp = lane >> 3;
    const int K = A.K, M = A.M;
    const int ksteps = (K + 31) >> 5;
    const int k8_last = (K >> 3) - 1;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const int c_begin = blockIdx.y * A.chunks_per_part;
    const int c_end = c_begin + A.chunks_per_part < A.chunks ? c_begin + A.chunks_per_part : A.chunks;

    // ---- this wave's tile of W
    const int tile = blockIdx.x * GT_WAVES + wave;
    const uint4* wp;
    if (FRAGW) {
        const int ntiles = EPI == GT_SWIGLU ? (A.N + 7) / 8 : (A.N + 15) / 16;
        wp = reinterpret_cast<const uint4*>(A.W) + (size_t)(tile < ntiles ? tile : ntiles - 1) * ksteps * 64 + lane;
    } else if (EPI == GT_SWIGLU) {   // rows 0..7 of the tile: gate rows of outputs 8 tile .., rows 8..15: their up rows
        const int o = tile * 8 + (r & 7);
        wp = reinterpret_cast<const uint4*>(A.W + (size_t)((o < A.N ? o : A.N - 1) + (r >> 3) * A.N) * A.ldw);
    } else {
        const int n = tile * 16 + r;
        wp = reinterpret_cast<const uint4*>(A.W + (size_t)(n < A.N ? n : A.N - 1) * A.ldw);
    }
    // Loads are unconditional 16-byte loads from clamped addresses; what lies beyond K or beyond M is replaced by
    // zeros on the X side, which makes the clamped W loads harmless.
#define GT_LOAD_W(DST_, CH_)                                                     \
    _Pragma("unroll") for (int s = 0; s < KS; ++s) {                             \
        if (FRAGW) {                                                             \
            const int st = (CH_) * KS + s;                                       \
            DST_[s] = wp[(size_t)(st < ksteps ? st : ksteps - 1) * 64];          \
        } else {                                                                 \
            const int k8 = (CH_) * (KC / 8) + s * 4 + q;                         \
            DST_[s] = wp[k8 <= k8_last ? k8 : k8_last];                          \
        }                                                                        \
    }
    // ---- staging of X: block b = (8 rows rb, line li) of the chunk; this wave takes blocks wave + 8 i (beyond the last
    // block it takes the last one again: the same bytes to the same place); a lane takes piece pp of row r8 of the
    // block.  The loads are unconditional and their values are looked at only when they are stored (a branch or a
    // select right after a load would make the wave wait for it there, with everything else that is in flight).
    // In LDS the piece lies where the operand's lane (row % 16, piece % 4) reads it.
#define GT_BLOCK(I_) ((BLOCKS % GT_WAVES == 0 || wave + GT_WAVES * (I_) < BLOCKS) ? wave + GT_WAVES * (I_) : BLOCKS - 1)
#define GT_X1(XV_, I_, CH_)                                                                                   \
    if (XPER > I_) {                                                                                          \
        const int b = GT_BLOCK(I_);                                                                           \
        const int row = (b / LINES) * 8 + r8;                                                                 \
        const int k8 = (CH_) * (KC / 8) + (b % LINES) * 8 + pp;                                               \
        XV_ = *reinterpret_cast<const uint4*>(A.X + (size_t)(row < M ? row : 0) * A.lda +                     \
                                              (size_t)(k8 <= k8_last ? k8 : k8_last) * 8);                    \
    }
#define GT_LOAD_X(CH_)                                                                                        \
    GT_X1(x0, 0, CH_) GT_X1(x1, 1, CH_) GT_X1(x2, 2, CH_) GT_X1(x3, 3, CH_)                                   \
    GT_X1(x4, 4, CH_) GT_X1(x5, 5, CH_) GT_X1(x6, 6, CH_) GT_X1(x7, 7, CH_)
#define GT_S1(XV_, I_, BUF_, CH_)                                                                             \
    if (XPER > I_) {                                                                                          \
        const int b = GT_BLOCK(I_);                                                                           \
        const int rb = b / LINES, li = b % LINES;                                                             \
        const bool ok = rb * 8 + r8 < M && (CH_) * (KC / 8) + li * 8 + pp <= k8_last;                         \
        const unsigned mk = ok ? 0xffffffffu : 0u;   /* (a select between two 16-byte structs goes through memory) */ \
        Xs[BUF_][2 * li + (pp >> 2)][rb >> 1][(pp & 3) * 16 + (rb & 1) * 8 + r8] =                            \
            make_uint4(XV_.x & mk, XV_.y & mk, XV_.z & mk, XV_.w & mk);                                       \
    }
#define GT_STORE_X(BUF_, CH_)                                                                                 \
    GT_S1(x0, 0, BUF_, CH_) GT_S1(x1, 1, BUF_, CH_) GT_S1(x2, 2, BUF_, CH_) GT_S1(x3, 3, BUF_, CH_)           \
    GT_S1(x4, 4, BUF_, CH_) GT_S1(x5, 5, BUF_, CH_) GT_S1(x6, 6, BUF_, CH_) GT_S1(x7, 7, BUF_, CH_)

    f32x4 acc[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
    uint4 x0 = zero, x1 = zero, x2 = zero, x3 = zero, x4 = zero, x5 = zero, x6 = zero, x7 = zero;
    uint4 wa[KS], wb[KS];
    GT_LOAD_X(c_begin)
    GT_LOAD_W(wa, c_begin)
    GT_STORE_X(0, c_begin)
    __syncthreads();
    // Two chunks an iteration, so that the W fragments in flight alternate between two sets of registers.  Inside a
    // chunk one half of the groups' X fragments is read from LDS while the other half is multiplied.
    constexpr int HA = (MG + 1) / 2, HB = MG - HA;
    uint4 ba[HA], bb[HB];
#define GT_READ_A(BUF_, S_) _Pragma("unroll") for (int g = 0; g < HA; ++g) ba[g] = Xs[BUF_][S_][g][lane];
#define GT_READ_B(BUF_, S_) _Pragma("unroll") for (int g = 0; g < HB; ++g) bb[g] = Xs[BUF_][S_][HA + g][lane];
#define GT_MUL_A(W_) _Pragma("unroll") for (int g = 0; g < HA; ++g) acc[g] = gt_mfma(W_, ba[g], acc[g]);
#define GT_MUL_B(W_) _Pragma("unroll") for (int g = 0; g < HB; ++g) acc[HA + g] = gt_mfma(W_, bb[g], acc[HA + g]);
#define GT_CHUNK(WCUR_, WNEXT_, CH_, BUF_)                                                                    \
    {                                                                                                         \
        {                                                                                                     \
            /* The next chunk's loads, unconditionally (after the last chunk: that one again, for nothing): behind a \
               branch the compiler could not count how many loads are younger than the fragments it is about to use \
               and would wait for most of them.  X first: the wait for it before the store below then leaves the W \
               loads, issued later, in flight */                                                              \
            const int nx = (CH_) + 1 < c_end ? (CH_) + 1 : c_end - 1;                                         \
            GT_LOAD_X(nx)                                                                                     \
            GT_LOAD_W(WNEXT_, nx)                                                                             \
        }                                                                                                     \
        __builtin_amdgcn_sched_barrier(0);                                                                    \
        GT_READ_A(BUF_, 0)                                                                                    \
        _Pragma("unroll") for (int s = 0; s < KS; ++s) {                                                      \
            GT_READ_B(BUF_, s)                                                                                \
            __builtin_amdgcn_sched_barrier(0);                                                                \
            GT_MUL_A(WCUR_[s])                                                                                \
            __builtin_amdgcn_sched_barrier(0);                                                                \
            if (s + 1 < KS) GT_READ_A(BUF_, s + 1)                                                            \
            __builtin_amdgcn_sched_barrier(0);                                                                \
            GT_MUL_B(WCUR_[s])                                                                                \
            __builtin_amdgcn_sched_barrier(0);                                                                \
        }                                                                                                     \
        if ((CH_) + 1 < c_end) GT_STORE_X((BUF_) ^ 1, (CH_) + 1)   /* its readers passed the barrier one chunk ago */ \
        __syncthreads();                                                                                      \
    }
    for (int ch = c_begin; ch < c_end; ch += 2) {
        GT_CHUNK(wa, wb, ch, 0)
        if (ch + 1 < c_end) GT_CHUNK(wb, wa, ch + 1, 1)
    }
#undef GT_CHUNK
#undef GT_READ_A
#undef GT_READ_B
#undef GT_MUL_A
#undef GT_MUL_B
#undef GT_BLOCK
#undef GT_LOAD_W
#undef GT_LOAD_X
#undef GT_X1
#undef GT_S1
#undef GT_STORE_X

    // acc[g][e] of lane (r, q): row 16 g + r of X, row 4 q + e of the tile
    if (EPI == GT_PARTS) {
        float* Cp = A.C + (size_t)blockIdx.y * A.part_stride;
        const int n = tile * 16 + q * 4;
#pragma unroll
        for (int g = 0; g < MG; ++g) {
            const int m = g * 16 + r;
            if (m >= M) continue;
            float* dst = Cp + (size_t)m * A.ldc + n;
            if (n + 3 < A.N && (A.ldc & 3) == 0) {
                *reinterpret_cast<f32x4*>(dst) = acc[g];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < A.N) dst[e] = acc[g][e];
            }
        }
    } else {
        // gate rows for q < 2, up rows for q >= 2: the lane 32 further on holds the up sums of this lane's outputs
        const int I = A.N;
        const int n = tile * 8 + q * 4;
        float bg[4] = {0.f, 0.f, 0.f, 0.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
        if (A.bias != nullptr && q < 2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int ne = n + e < I ? n + e : I - 1;
                bg[e] = to_f32(A.bias[ne]);
                bu[e] = to_f32(A.bias[ne + I]);
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
            bf16* dst = A.act + (size_t)m * A.ld_act + n;
            if (n + 3 < I && (A.ld_act & 3) == 0 && ((uintptr_t)A.act & 7) == 0) {
                *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(o);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < I) dst[e] = o[e];
            }
        }
    }
}

extern "C" int ilm_gemm_tall_max_rows() { return 208; }

template <int EPI>
static void gt_launch(const GtArgs& a, int kc, dim3 grid, int frag_w, hipStream_t stream) {
#define GT_GO(MG_, KC_)                                                                                        \
    if (frag_w) gemm_tall_kernel<MG_, KC_, true, EPI><<<grid, GT_THREADS, 0, stream>>>(a);                     \
    else gemm_tall_kernel<MG_, KC_, false, EPI><<<grid, GT_THREADS, 0, stream>>>(a)
#define GT_KC(MG_) if (kc == 64) { GT_GO(MG_, 64); } else { GT_GO(MG_, 128); }
    switch ((a.M + 15) / 16) {
        case 2: GT_KC(2) break;
        case 3: GT_KC(3) break;
        case 4: GT_KC(4) break;
        case 5: GT_KC(5) break;
        case 6: GT_KC(6) break;
        case 7: GT_KC(7) break;
        case 8: GT_KC(8) break;
        case 9: GT_KC(9) break;
        case 10: GT_KC(10) break;
        case 11: GT_KC(11) break;
        case 12: GT_KC(12) break;
        default: GT_KC(13) break;
    }
#undef GT_KC
#undef GT_GO
}

static int gt_check(const char* what, int M, int N, int K, int kc, const void* X, int lda, const void* W, int ldw, int frag_w) {
    ILM_REQUIRE(M > 16 && M <= 208 && N > 0 && K > 0, "%s: needs 17 <= M <= 208, got M=%d N=%d K=%d", what, M, N, K);
    ILM_REQUIRE(kc == 64 || kc == 128, "%s: chunks of %d k (64 or 128)", what, kc);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && lda >= K && (frag_w || (ldw % 8 == 0 && ldw >= K)), "%s: K=%d lda=%d ldw=%d", what,
                K, lda, ldw);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "%s: operands must be 16-byte aligned", what);
    return 0;
}

// C: float [kb][M][ldc] with c_part_stride elements between the parts; part y covers chunks_per_part chunks of kc k
// (64 or 128) from y * chunks_per_part on, kb = ceil(ceil(K / kc) / chunks_per_part).
// frag_w != 0: W is the weight in fragment order, tiles of 16 consecutive rows (ldw is not used).
extern "C" int ilm_gemm_tall(void* C, int ldc, long c_part_stride, int kb, int chunks_per_part, int kc, const void* W, int ldw,
                             int M, int N, int K, const void* X, int lda, int frag_w, hipStream_t stream) {
    if (gt_check("gemm_tall", M, N, K, kc, X, lda, W, ldw, frag_w)) return -1;
    GtArgs a = {};
    a.X = (const bf16*)X; a.W = (const bf16*)W; a.M = M; a.N = N; a.K = K; a.lda = lda; a.ldw = ldw;
    a.chunks = (K + kc - 1) / kc;
    a.chunks_per_part = chunks_per_part;
    ILM_REQUIRE(chunks_per_part > 0 && kb == (a.chunks + chunks_per_part - 1) / chunks_per_part && kb <= 65535,
                "gemm_tall: %d parts of %d chunks do not cover the %d chunks of K=%d", kb, chunks_per_part, a.chunks, K);
    ILM_REQUIRE(ldc >= N && ((uintptr_t)C & 15) == 0, "gemm_tall: ldc=%d", ldc);
    a.C = (float*)C; a.ldc = ldc; a.part_stride = (size_t)c_part_stride;
    gt_launch<GT_PARTS>(a, kc, dim3((N + GT_NT - 1) / GT_NT, kb), frag_w, stream);
    ILM_LAUNCH_CHECK("gemm_tall");
    return 0;
}

// act [M, ld_act] = silu(X Wg^T + bg) * (X Wu^T + bu) with W = [Wg; Wu] of 2 I rows (bias of 2 I entries or null); kc: k a
// chunk (64 or 128).  frag_w != 0: W is the weight in fragment order with tiles of 8 gate + 8 up rows (ldw is not used).
extern "C" int ilm_gemm_tall_swiglu(void* act, int ld_act, const void* X, int lda, const void* W, int ldw, const void* bias,
                                    int M, int I, int K, int kc, int frag_w, hipStream_t stream) {
    if (gt_check("gemm_tall_swiglu", M, I, K, kc, X, lda, W, ldw, frag_w)) return -1;
    ILM_REQUIRE(ld_act >= I, "gemm_tall_swiglu: ld_act=%d", ld_act);
    GtArgs a = {};
    a.X = (const bf16*)X; a.W = (const bf16*)W; a.bias = (const bf16*)bias; a.M = M; a.N = I; a.K = K; a.lda = lda; a.ldw = ldw;
    a.chunks = (K + kc - 1) / kc;
    a.chunks_per_part = a.chunks;
    a.act = (bf16*)act; a.ld_act = ld_act;
    gt_launch<GT_SWIGLU>(a, kc, dim3((I + GT_NT / 2 - 1) / (GT_NT / 2), 1), frag_w, stream);
    ILM_LAUNCH_CHECK("gemm_tall_swiglu");
    return 0;
}
