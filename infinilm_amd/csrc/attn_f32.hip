// Paged attention of the 32-bit path on the float matrix instruction (v_mfma_f32_16x16x4_f32: IEEE float
// products and sums, no reduced-precision mode).  Contract as in attn_basic.hip: token t of request seg[t]
// at position pos[t] sees its request's keys [lo, pos[t]] through block_tables.
//
// A wave serves one token and up to 16 query heads that share a KV head: the heads are the columns of the
// matrix instruction, so a key or value is read once for all of them (the plain kernel read it once a
// head).  Keys are taken in chunks of FA_CHUNK keys aligned to the absolute key index.  A chunk gives a
// partial result from a fresh start: scores of its 8 tiles of 16 keys, their maximum, the exponentials,
// their sum, and the weighted values; the chunks' partial results are folded in ascending order.  So the
// order of every sum is fixed by (request, position) alone, whichever of the two launch shapes runs: one
// wave that walks all chunks of its token and folds as it goes (many tokens), or one wave a chunk that
// writes its partial result to a workspace, and a fold kernel (few tokens over long contexts).
//
// Score product: K tile on the A side (16 keys x 4 dims), Q on the B side (4 dims x 16 heads); a lane
// (r = lane % 16, q = lane / 16) loads 16 bytes of key r (dims 16j + 4q ...) and feeds four instructions,
// one an element.  The result leaves lane (r, q) with the scores of head r for keys 4q .. 4q+3 of the
// tile, which is the B-side layout of the second product (V^T tile of 16 dims x 4 keys on the A side,
// values transposed in the cache: 16 bytes are four consecutive keys of one dim): no exchange between lanes.
// Needs head sizes in steps of 16 up to 256, pages that are multiples of 4 keys, 16-byte aligned rows.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;

#define FA_CHUNK 128
#define FA_TILES (FA_CHUNK / 16)
#define FA_WS_PAD 4   // a partial result is d outputs, its maximum, its sum and two unused floats (16-byte rows)

__device__ __forceinline__ f32x4 fa_mfma(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// (M, L, ACC) <- fold of (M, L, ACC) and a chunk's (m, l, acc): explicit multiply-adds, the same in both
// launch shapes and in the fold kernel
__device__ __forceinline__ void fa_fold_scales(float& M, float& L, float m, float l, float& a, float& b) {
    const float Mn = fmaxf(M, m);
    a = expf(M - Mn);
    b = expf(m - Mn);
    L = fmaf(L, a, l * b);
    M = Mn;
}

// DT: head size / 16.  !SPLIT: gridDim.z == 1 and the wave walks all chunks; SPLIT: blockIdx.z is the
// chunk and the partial result goes to ws[((t * nh + h) * gridDim.z + chunk) * (d + FA_WS_PAD)].
template <int DT, bool SPLIT>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(DT <= 8 ? 2 : 1)))
attn_f32_kernel(float* __restrict__ out, float* __restrict__ ws, const float* __restrict__ qp, const float* __restrict__ kc,
                const float* __restrict__ vc, const int* __restrict__ block_tables, const int* __restrict__ seg,
                const int* __restrict__ pos, int nh, int nkv, int nsub, int page, int max_blocks, int q_stride,
                int out_stride, float scale, int window) {
    constexpr int d = DT * 16;
    // tiles of keys (and of values) in flight: two, or one where the running result of the wave that walks all
    // chunks leaves no registers for the second (another wave of the SIMD then covers the wait)
    constexpr int NB = (!SPLIT && DT > 6) ? 1 : 2;
    const int t = blockIdx.x, lane = threadIdx.x, r = lane & 15, q = lane >> 4;
    const int G = nh / nkv;
    const int kvh = blockIdx.y / nsub, sub = blockIdx.y % nsub;
    const int heads = (G - sub * 16 < 16) ? G - sub * 16 : 16;
    const int h = kvh * G + sub * 16 + (r < heads ? r : heads - 1);
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    int c_first = lo / FA_CHUNK, c_last = p / FA_CHUNK;
    if (SPLIT) {
        if ((int)blockIdx.z < c_first || (int)blockIdx.z > c_last) return;   // the fold reads only the chunks the token sees
        c_first = c_last = blockIdx.z;
    }
    const int* bt = block_tables + (size_t)seg[t] * max_blocks;
    // the token's queries: lane (r, q) holds dims 16j + 4q .. + 3 of head r
    float4 qf[DT];
    {
        const float4* qrow = reinterpret_cast<const float4*>(qp + (size_t)t * q_stride + (size_t)h * d);
#pragma unroll
        for (int j = 0; j < DT; ++j) qf[j] = qrow[4 * j + q];
    }
    float M = -INFINITY, L = 0.f;
    f32x4 ACC[SPLIT ? 1 : DT];
#pragma unroll
    for (int i = 0; i < (SPLIT ? 1 : DT); ++i) ACC[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int c = c_first; c <= c_last; ++c) {
        const int k_lo = lo > c * FA_CHUNK ? lo : c * FA_CHUNK;
        const int k_hi = p < c * FA_CHUNK + FA_CHUNK - 1 ? p : c * FA_CHUNK + FA_CHUNK - 1;
        // tiles with a key the token sees: t_first .. t_last.  Tiles before t_first (under a window only) are
        // walked with every key masked, which adds exact zeros: the buffers alternate by tile number
        const int t_first = (k_lo - c * FA_CHUNK) >> 4, t_last = (k_hi - c * FA_CHUNK) >> 4;

        // ---- scores of the chunk's tiles; the next tile's keys are on their way while one is multiplied
        f32x4 S[FA_TILES];
        float4 kf[NB][DT];
#define FA_LOAD_K(BUF_, KT_)                                                                                  \
        {                                                                                                     \
            int key = c * FA_CHUNK + (KT_) * 16 + r;                                                          \
            key = key < k_lo ? k_lo : (key > k_hi ? k_hi : key);   /* rows the token does not see: a row it sees */ \
            const int pg = bt[key / page];                                                                    \
            const float4* krow = reinterpret_cast<const float4*>(kc + (((size_t)pg * nkv + kvh) * page + (key % page)) * d); \
            _Pragma("unroll") for (int j = 0; j < DT; ++j) kf[BUF_][j] = krow[4 * j + q];                      \
        }
        if (NB == 2) FA_LOAD_K(0, 0)
#pragma unroll
        for (int kt = 0; kt < FA_TILES; ++kt) {
            S[kt] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            if (kt > t_last) continue;
            if (NB == 1) FA_LOAD_K(0, kt)
            else if (kt + 1 < FA_TILES && kt < t_last) FA_LOAD_K((kt + 1) & (NB - 1), kt + 1)
            __builtin_amdgcn_sched_barrier(0);
            f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < DT; ++j) {
                s = fa_mfma(kf[kt & (NB - 1)][j].x, qf[j].x, s);
                s = fa_mfma(kf[kt & (NB - 1)][j].y, qf[j].y, s);
                s = fa_mfma(kf[kt & (NB - 1)][j].z, qf[j].z, s);
                s = fa_mfma(kf[kt & (NB - 1)][j].w, qf[j].w, s);
            }
            const int key0 = c * FA_CHUNK + kt * 16 + 4 * q;   // element e is the score of key key0 + e
#pragma unroll
            for (int e = 0; e < 4; ++e) S[kt][e] = (key0 + e >= k_lo && key0 + e <= k_hi) ? s[e] * scale : -INFINITY;
            __builtin_amdgcn_sched_barrier(0);
        }
#undef FA_LOAD_K
        // ---- maximum, exponentials and their sum per head (a head's scores lie in the four lanes r, r+16, r+32, r+48)
        float m = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < FA_TILES; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) m = fmaxf(m, S[kt][e]);
        m = fmaxf(m, __shfl_xor(m, 16, 64));
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        float l = 0.f;
#pragma unroll
        for (int kt = 0; kt < FA_TILES; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                S[kt][e] = expf(S[kt][e] - m);   // keys the token does not see: exp(-inf) = 0
                l += S[kt][e];
            }
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);

        // ---- weighted values: V^T tiles of 16 dims x 4 keys on the A side, the exponentials on the B side
        f32x4 acc[DT];
#pragma unroll
        for (int i = 0; i < DT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        float4 vf[NB][DT];
#define FA_LOAD_V(BUF_, KT_)                                                                                   \
        {                                                                                                      \
            int gk = c * FA_CHUNK + (KT_) * 16 + 4 * q;   /* the lane's four keys; groups wholly outside: a group inside */ \
            if (gk > k_hi) gk = k_hi & ~3;                                                                     \
            if (gk + 3 < k_lo) gk = k_lo & ~3;                                                                 \
            const int pg = bt[gk / page];                                                                      \
            const float* vbase = vc + ((size_t)pg * nkv + kvh) * d * page + (gk % page);                       \
            _Pragma("unroll") for (int i = 0; i < DT; ++i)                                                     \
                vf[BUF_][i] = *reinterpret_cast<const float4*>(vbase + (size_t)(16 * i + r) * page);           \
        }
        if (NB == 2) FA_LOAD_V(0, 0)
#pragma unroll
        for (int kt = 0; kt < FA_TILES; ++kt) {
            if (kt > t_last) continue;
            if (NB == 1) FA_LOAD_V(0, kt)
            else if (kt + 1 < FA_TILES && kt < t_last) FA_LOAD_V((kt + 1) & (NB - 1), kt + 1)
            __builtin_amdgcn_sched_barrier(0);
            // values of keys the token does not see may be anything (pages are not cleared): they count as zeros
            const int key0 = c * FA_CHUNK + kt * 16 + 4 * q;
            const bool edge = (kt <= t_first || kt == t_last);
            const bool ok0 = !edge || (key0 >= k_lo && key0 <= k_hi), ok1 = !edge || (key0 + 1 >= k_lo && key0 + 1 <= k_hi);
            const bool ok2 = !edge || (key0 + 2 >= k_lo && key0 + 2 <= k_hi), ok3 = !edge || (key0 + 3 >= k_lo && key0 + 3 <= k_hi);
            const f32x4 pw = S[kt];
#define FA_MUL_V(BUF_)                                                                      \
            _Pragma("unroll") for (int i = 0; i < DT; ++i) {                                \
                const float4 v = vf[BUF_][i];                                               \
                acc[i] = fa_mfma(ok0 ? v.x : 0.f, pw[0], acc[i]);                           \
                acc[i] = fa_mfma(ok1 ? v.y : 0.f, pw[1], acc[i]);                           \
                acc[i] = fa_mfma(ok2 ? v.z : 0.f, pw[2], acc[i]);                           \
                acc[i] = fa_mfma(ok3 ? v.w : 0.f, pw[3], acc[i]);                           \
            }
            FA_MUL_V(kt & (NB - 1))
#undef FA_MUL_V
            __builtin_amdgcn_sched_barrier(0);
        }
#undef FA_LOAD_V
        // acc[i][e] of lane (r, q): head r, dim 16 i + 4 q + e
        if (SPLIT) {
            if (r < heads) {
                float* dst = ws + (((size_t)t * nh + h) * gridDim.z + c) * (d + FA_WS_PAD);
#pragma unroll
                for (int i = 0; i < DT; ++i) *reinterpret_cast<f32x4*>(dst + 16 * i + 4 * q) = acc[i];
                if (q == 0) {
                    dst[d] = m;
                    dst[d + 1] = l;
                }
            }
            return;
        }
        float a, b;
        fa_fold_scales(M, L, m, l, a, b);
#pragma unroll
        for (int i = 0; i < (SPLIT ? 0 : DT); ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) ACC[i][e] = fmaf(ACC[i][e], a, acc[i][e] * b);
    }
    if (!SPLIT && r < heads) {
        float* orow = out + (size_t)t * out_stride + (size_t)h * d;
        const float inv = 1.0f / L;
#pragma unroll
        for (int i = 0; i < (SPLIT ? 0 : DT); ++i) {
            f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = ACC[i][e] * inv;
            *reinterpret_cast<f32x4*>(orow + 16 * i + 4 * q) = o;
        }
    }
}

// Folds the chunks' partial results of one (token, head) in ascending order, as the one-wave shape does: a
// thread a dim (the block has as many waves as the head has 64s of dims), every thread the scalars.  The
// loads of FA_FOLD_AHEAD chunks are in flight together; the fold itself stays one chain in chunk order.
// A token whose chunks do not all lie inside the workspace (the caller's bound was too small) gets a row of
// NaNs instead of a silently wrong one.
#define FA_FOLD_AHEAD 8
__global__ void __launch_bounds__(256)
attn_f32_fold_kernel(float* __restrict__ out, const float* __restrict__ ws, const int* __restrict__ pos, int nh, int d,
                     int nchunks, int out_stride, int window) {
    const int t = blockIdx.x, h = blockIdx.y, dim = threadIdx.x;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    float* orow = out + (size_t)t * out_stride + (size_t)h * d;
    if (p / FA_CHUNK > nchunks - 1) {
        if (dim < d) orow[dim] = __int_as_float(0x7fc00000);
        return;
    }
    const int dimc = dim < d ? dim : d - 1;
    const int c_last = p / FA_CHUNK;
    const float* base = ws + ((size_t)t * nh + h) * nchunks * (d + FA_WS_PAD);
    float M = -INFINITY, L = 0.f, ACC = 0.f;
    for (int c0 = lo / FA_CHUNK; c0 <= c_last; c0 += FA_FOLD_AHEAD) {
        float mm[FA_FOLD_AHEAD], ll[FA_FOLD_AHEAD], av[FA_FOLD_AHEAD];
#pragma unroll
        for (int u = 0; u < FA_FOLD_AHEAD; ++u) {
            const int c = c0 + u <= c_last ? c0 + u : c_last;
            const float* src = base + (size_t)c * (d + FA_WS_PAD);
            mm[u] = src[d];
            ll[u] = src[d + 1];
            av[u] = src[dimc];
        }
#pragma unroll
        for (int u = 0; u < FA_FOLD_AHEAD; ++u) {
            if (c0 + u <= c_last) {
                float a, b;
                fa_fold_scales(M, L, mm[u], ll[u], a, b);
                ACC = fmaf(ACC, a, av[u] * b);
            }
        }
    }
    if (dim < d) orow[dim] = ACC * (1.0f / L);
}

extern "C" int ilm_attn_f32_chunk() { return FA_CHUNK; }
extern "C" int ilm_attn_f32_ws_row(int d) { return d + FA_WS_PAD; }

// ws: null (one wave walks all chunks of its token), or float [T][nh][nchunks][d + 4] with
// nchunks >= ceil((largest position + 1) / ilm_attn_f32_chunk()): one wave a chunk, then the fold.
extern "C" int ilm_attn_f32(void* out, void* ws, int nchunks, const void* q, const void* kc, const void* vc,
                            const void* block_tables, const void* seg, const void* pos, int T_, int nh, int nkv, int d,
                            int page, int max_blocks, int q_stride, int out_stride, float scale, int window,
                            hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv > 0 && d > 0 && page > 0 && max_blocks > 0, "attn_f32: bad sizes");
    ILM_REQUIRE(nh % nkv == 0, "attn_f32: %d query heads do not divide into %d groups", nh, nkv);
    ILM_REQUIRE(d % 16 == 0 && d <= 256, "attn_f32: head size %d is no multiple of 16 up to 256", d);
    ILM_REQUIRE(page % 4 == 0, "attn_f32: pages of %d keys are no multiple of 4", page);
    ILM_REQUIRE(q_stride % 4 == 0 && out_stride % 4 == 0 && ((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 15) == 0
                    && ((uintptr_t)kc & 15) == 0 && ((uintptr_t)vc & 15) == 0 && (ws == nullptr || ((uintptr_t)ws & 15) == 0),
                "attn_f32: rows must be 16-byte aligned");
    ILM_REQUIRE(ws == nullptr || (nchunks >= 1 && nchunks <= 65535), "attn_f32: %d chunks", nchunks);
    const int G = nh / nkv, nsub = (G + 15) / 16;
    ILM_REQUIRE((long long)nkv * nsub <= 65535 && nh <= 65535, "attn_f32: too many heads");
    dim3 grid(T_, nkv * nsub, ws != nullptr ? nchunks : 1);
#define FA_ARGS (float*)out, (float*)ws, (const float*)q, (const float*)kc, (const float*)vc, (const int*)block_tables, \
                (const int*)seg, (const int*)pos, nh, nkv, nsub, page, max_blocks, q_stride, out_stride, scale, window
#define FA_CASE(DT_)                                                                        \
    case DT_:                                                                               \
        if (ws != nullptr) attn_f32_kernel<DT_, true><<<grid, 64, 0, stream>>>(FA_ARGS);    \
        else attn_f32_kernel<DT_, false><<<grid, 64, 0, stream>>>(FA_ARGS);                 \
        break;
    switch (d / 16) {
        FA_CASE(1) FA_CASE(2) FA_CASE(3) FA_CASE(4) FA_CASE(5) FA_CASE(6) FA_CASE(7) FA_CASE(8)
        FA_CASE(9) FA_CASE(10) FA_CASE(11) FA_CASE(12) FA_CASE(13) FA_CASE(14) FA_CASE(15) FA_CASE(16)
        default: ILM_REQUIRE(false, "attn_f32: head size %d", d);
    }
#undef FA_CASE
#undef FA_ARGS
    ILM_LAUNCH_CHECK("attn_f32");
    if (ws != nullptr) {
        attn_f32_fold_kernel<<<dim3(T_, nh), 64 * ((d + 63) / 64), 0, stream>>>((float*)out, (const float*)ws, (const int*)pos, nh, d, nchunks,
                                                              out_stride, window);
        ILM_LAUNCH_CHECK("attn_f32_fold");
    }
    return 0;
}
