// Products of 17 to 64 rows of X (bfloat16) with W [N, K] streamed once, every output with one owner.
//
// A workgroup of 8 waves takes NT tiles of 16 rows of W and all rows of X; the waves split the workgroup's
// range of K and their partial tiles meet in LDS, where the thread that reduces an output applies the
// epilogue (plain store, float parts of a K split over workgroups, SwiGLU of a gate and an up row, rotation
// and cache write of a q/k/v pair, residual sum and half a norm).
//
// How operands reach the matrix instruction decides the speed here.  A load that hands a lane its fragment
// directly (lane (r, q): 16 bytes of row r) touches 16 rows and half a 128-byte line of each: a compute
// unit takes in about 36 GB/s that way, 9 TB/s over the chip, whatever the source (measured with reads that
// hit L2).  A load in which 8 lanes cover one whole line (8 rows x 128 bytes an instruction) runs at 130
// GB/s a unit.  W alone, read once from memory, lives with the first form; but X is read by every workgroup,
// from the L2s, so here both go the second way: a wave loads a stage (64 k = one line a row) of its own X
// rows and W rows in whole lines, parks it in a private piece of LDS (16-byte chunks swizzled by row, no
// bank conflicts either way) and reads the fragments back.  The LDS traffic stays inside the wave: no
// workgroup barrier in the loop, the waves drift apart as their loads arrive.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define GW_WAVES 8
#define GW_STAGE 64   // k a stage: 128 bytes a row

__device__ __forceinline__ f32x4 gw_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// orders a wave's LDS writes before its LDS reads of other lanes' data (and the reverse) for the compiler;
// the hardware runs a wave's LDS instructions in order
__device__ __forceinline__ void gw_wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// LDS of a workgroup: the waves' stages during the product, their partial tiles after it
template <int MG, int NT>
struct GwLds {
    static constexpr int STAGE_U4 = (MG + NT) * 16 * 8;                  // uint4 a wave: rows x 8 chunks
    static constexpr int STAGE_BYTES = GW_WAVES * STAGE_U4 * 16;
    static constexpr int PART_BYTES = NT * MG * GW_WAVES * 64 * 16;
    static constexpr int BYTES = STAGE_BYTES > PART_BYTES ? STAGE_BYTES : PART_BYTES;
};

// The wave's share of the product: acc[t][g] += W tile t x X group g over k in [k_begin, k_end).
// wrow[j]: the W row this lane loads in load j (tile j / 2, row 8 (j % 2) + lane / 8 of the tile).
template <int MG, int NT>
__device__ __forceinline__ void gw_product(f32x4 (&acc)[NT][MG], const bf16* __restrict__ X, int lda, int M,
                                           const bf16* __restrict__ W, int ldw, const int (&wrow)[2 * NT], int k_begin,
                                           int k_end, uint4* __restrict__ stage) {
    const int lane = threadIdx.x & 63;
    const int row8 = lane >> 3, c = lane & 7;      // loader: 8 lanes a row, 16 bytes each
    const int r = lane & 15, q = lane >> 4;        // matrix instruction: lane (r, q) holds row r, k 8 q .. 8 q + 7 of a step
    const int swz = (r >> 1) & 7;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const bf16* xsrc[2 * MG];
    const bf16* wsrc[2 * NT];
    int xdst[2 * MG], wdst[2 * NT];
#pragma unroll
    for (int j = 0; j < 2 * MG; ++j) {
        const int row = 8 * j + row8;
        xsrc[j] = X + (size_t)(row < M ? row : M - 1) * lda;
        xdst[j] = row * 8 + (c ^ ((row >> 1) & 7));
    }
#pragma unroll
    for (int j = 0; j < 2 * NT; ++j) {
        const int row = 8 * j + row8;
        wsrc[j] = W + (size_t)wrow[j] * ldw;
        wdst[j] = MG * 128 + row * 8 + (c ^ ((row >> 1) & 7));
    }
    const int stages = (k_end - k_begin + GW_STAGE - 1) / GW_STAGE;
    uint4 gx[2][2 * MG], gw[2][2 * NT];
#define GW_LOAD(BUF_, S_)                                                                         \
    {                                                                                             \
        const int k = k_begin + (S_) * GW_STAGE + 8 * c;                                          \
        const bool ok = k < k_end;                                                                \
        const int kc = ok ? k : k_end - 8;                                                        \
        _Pragma("unroll") for (int j = 0; j < 2 * NT; ++j)                                        \
            gw[BUF_][j] = *reinterpret_cast<const uint4*>(wsrc[j] + kc);                          \
        _Pragma("unroll") for (int j = 0; j < 2 * MG; ++j)                                        \
            gx[BUF_][j] = *reinterpret_cast<const uint4*>(xsrc[j] + kc);                          \
        if (!ok) {   /* beyond the range: zeros on the X side */                                  \
            _Pragma("unroll") for (int j = 0; j < 2 * MG; ++j) gx[BUF_][j] = zero;                \
        }                                                                                         \
    }
#define GW_STEP(BUF_, S_)                                                                         \
    {                                                                                             \
        _Pragma("unroll") for (int j = 0; j < 2 * MG; ++j) stage[xdst[j]] = gx[BUF_][j];          \
        _Pragma("unroll") for (int j = 0; j < 2 * NT; ++j) stage[wdst[j]] = gw[BUF_][j];          \
        gw_wave_sync();                                                                           \
        if ((S_) + 2 < stages) GW_LOAD(BUF_, (S_) + 2)                                            \
        uint4 fa[2][NT], fb[2][MG];                                                               \
        _Pragma("unroll") for (int h = 0; h < 2; ++h) {                                           \
            _Pragma("unroll") for (int g = 0; g < MG; ++g)                                        \
                fb[h][g] = stage[(16 * g + r) * 8 + ((4 * h + q) ^ swz)];                         \
            _Pragma("unroll") for (int t = 0; t < NT; ++t)                                        \
                fa[h][t] = stage[MG * 128 + (16 * t + r) * 8 + ((4 * h + q) ^ swz)];              \
        }                                                                                         \
        gw_wave_sync();                                                                           \
        _Pragma("unroll") for (int h = 0; h < 2; ++h)                                             \
            _Pragma("unroll") for (int g = 0; g < MG; ++g)                                        \
                _Pragma("unroll") for (int t = 0; t < NT; ++t)                                    \
                    acc[t][g] = gw_mfma(fa[h][t], fb[h][g], acc[t][g]);                           \
    }
    if (stages > 0) GW_LOAD(0, 0)
    if (stages > 1) GW_LOAD(1, 1)
    for (int s = 0; s < stages; s += 2) {
        GW_STEP(0, s)
        if (s + 1 < stages) GW_STEP(1, s + 1)
    }
#undef GW_LOAD
#undef GW_STEP
}

// the wave's range of k inside the workgroup's [k_lo, k_hi): whole stages, spread evenly
__device__ __forceinline__ void gw_wave_range(int k_lo, int k_hi, int& k_begin, int& k_end) {
    const int wave = threadIdx.x >> 6;
    const int stages = (k_hi - k_lo + GW_STAGE - 1) / GW_STAGE;
    const int per = (stages + GW_WAVES - 1) / GW_WAVES;
    k_begin = k_lo + wave * per * GW_STAGE;
    k_end = k_begin + per * GW_STAGE;
    if (k_end > k_hi) k_end = k_hi;
    if (k_begin > k_hi) k_begin = k_hi;
}

template <int MG, int NT>
__device__ __forceinline__ void gw_park(const f32x4 (&acc)[NT][MG], float* part) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g)
            *reinterpret_cast<f32x4*>(part + ((((size_t)t * MG + g) * GW_WAVES + wave) * 64 + lane) * 4) = acc[t][g];
}

// sum over the waves of output (tile t, group g, lane l, element e): row 16 g + l % 16 of X, row 4 (l / 16) + e of the tile
template <int MG>
__device__ __forceinline__ float gw_reduce(const float* part, int t, int g, int l, int e) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < GW_WAVES; ++w) v += part[((((size_t)t * MG + g) * GW_WAVES + w) * 64 + l) * 4 + e];
    return v;
}

// ---- plain store: C[kb][m][n] = alpha * (X W^T + bias) over the workgroup's K range kb (float parts when K is
// split over blockIdx.y, else one result in float or bfloat16)
template <int MG, int NT>
__global__ void __launch_bounds__(GW_WAVES * 64)
gemm_wide_plain_kernel(void* __restrict__ C, int ldc, long part_stride, int out_f32, const bf16* __restrict__ X,
                       const bf16* __restrict__ W, const bf16* __restrict__ bias, int M, int N, int K, int lda, int ldw,
                       int kspan, float alpha) {
    __shared__ __align__(16) unsigned char lds[GwLds<MG, NT>::BYTES];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n0 = blockIdx.x * (16 * NT);
    int wrow[2 * NT];
#pragma unroll
    for (int j = 0; j < 2 * NT; ++j) {
        const int n = n0 + 8 * j + (lane >> 3);
        wrow[j] = n < N ? n : N - 1;
    }
    const int k_lo = blockIdx.y * kspan, k_hi = (k_lo + kspan < K) ? k_lo + kspan : K;
    int k_begin, k_end;
    gw_wave_range(k_lo, k_hi, k_begin, k_end);
    f32x4 acc[NT][MG];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};
    gw_product<MG, NT>(acc, X, lda, M, W, ldw, wrow, k_begin, k_end,
                       reinterpret_cast<uint4*>(lds) + wave * GwLds<MG, NT>::STAGE_U4);
    __syncthreads();   // every wave has left its stage: the partial tiles take the same LDS
    float* part = reinterpret_cast<float*>(lds);
    gw_park<MG, NT>(acc, part);
    __syncthreads();
    for (int et = threadIdx.x; et < NT * MG * 256; et += GW_WAVES * 64) {
        const int e = et & 3, l = (et >> 2) & 63, tg = et >> 8;
        const int t = tg / MG, g = tg % MG;
        const int m = 16 * g + (l & 15), n = n0 + 16 * t + 4 * (l >> 4) + e;
        if (m >= M || n >= N) continue;
        float v = gw_reduce<MG>(part, t, g, l, e);
        if (bias != nullptr && blockIdx.y == 0) v += to_f32(bias[n]);
        v *= alpha;
        if (out_f32) reinterpret_cast<float*>(C)[(size_t)blockIdx.y * part_stride + (size_t)m * ldc + n] = v;
        else reinterpret_cast<bf16*>(C)[(size_t)m * ldc + n] = from_f32<bf16>(v);
    }
}

extern "C" int ilm_gemm_wide_stage() { return GW_STAGE; }

// C: float [parts][M][ldc] (parts = ceil(K / kspan), part_stride floats apart; bias in part 0) or, with
// kspan >= K, one float or bfloat16 result [M][ldc].  17 <= M <= 64.
extern "C" int ilm_gemm_wide(void* C, int ldc, long part_stride, int out_f32, const void* X, int lda, const void* W, int ldw,
                             const void* bias, int M, int N, int K, int kspan, float alpha, int tiles, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_wide: needs 1 <= M <= 64, got M=%d N=%d K=%d", M, N, K);
    ILM_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldc >= N,
                "gemm_wide: K=%d lda=%d ldw=%d ldc=%d", K, lda, ldw, ldc);
    ILM_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_wide: operands must be 16-byte aligned");
    ILM_REQUIRE(kspan > 0 && kspan % GW_STAGE == 0, "gemm_wide: a K range of %d is no multiple of %d", kspan, GW_STAGE);
    const int parts = (K + kspan - 1) / kspan;
    ILM_REQUIRE(parts == 1 || out_f32, "gemm_wide: parts of a split K are float");
    ILM_REQUIRE(parts <= 65535, "gemm_wide: %d parts", parts);
    ILM_REQUIRE(tiles == 2 || tiles == 4, "gemm_wide: %d tiles a workgroup", tiles);
    const int mg = (M + 15) / 16;
#define GW_PLAIN(MG_, NT_)                                                                                              \
    gemm_wide_plain_kernel<MG_, NT_><<<dim3((N + 16 * NT_ - 1) / (16 * NT_), parts), GW_WAVES * 64, 0, stream>>>(       \
        C, ldc, part_stride, out_f32, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, N, K, lda, ldw, kspan, alpha)
    if (tiles == 2) {
        switch (mg) {
            case 1: GW_PLAIN(1, 2); break;
            case 2: GW_PLAIN(2, 2); break;
            case 3: GW_PLAIN(3, 2); break;
            default: GW_PLAIN(4, 2); break;
        }
    } else {
        switch (mg) {
            case 1: GW_PLAIN(1, 4); break;
            case 2: GW_PLAIN(2, 4); break;
            case 3: GW_PLAIN(3, 4); break;
            default: GW_PLAIN(4, 4); break;
        }
    }
#undef GW_PLAIN
    ILM_LAUNCH_CHECK("gemm_wide");
    return 0;
}
