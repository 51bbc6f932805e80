// Paged attention on the matrix cores (bfloat16 in, float softmax and accumulation).
//
// Same contract as attn_basic.hip.  Two kernels: single tokens (decoding) over key chunks, below,
// and tiles of consecutive tokens of one request (portions of prompts), further down.
//
// Single tokens: `rows` (optional) lists the token rows to serve.  A workgroup of 4 waves serves one
// token and one group of up to 16 query heads that share a KV head, over one chunk of `span` keys
// (a multiple of ATT_STEP = 128, chosen by the caller so that the launch fills the chip: short
// chunks for few tokens, long ones for many).  The chunk is walked in steps of 128 keys, 32 a wave,
// the loads of the next step in flight while this one is multiplied; the four waves' partial
// results are merged through LDS.  Chunks are aligned to absolute key index.  With more than one
// chunk the partial results (max, sum, unnormalised output) go to a workspace and a second kernel
// merges them in chunk order.  For a given chunk length the result depends on (request, position)
// alone; another chunk length changes the order of summation, not more.
//
// Per 32 keys:  S^T[keys x heads] = K Q^T   (v_mfma_f32_16x16x32_bf16, K rows on the A side, read
//                                            straight from the cache; d is the reduced dimension)
//               online softmax in float, per head = per lane column
//               O^T[d x heads] += V^T P^T   (V is cached transposed, [d][page], so that 8
//                                            consecutive keys of one dim are one 16-byte load)
// The rows of the two S tiles are assigned to keys so that each lane ends up with the
// probabilities of 8 consecutive keys: they feed the second product without leaving registers.
// Loads are unconditional 16-byte loads from clamped addresses, masked afterwards.
// Needs: head size a multiple of 16 up to 128, page size a multiple of 16.
#include "common.h"
#include "no_alloc.h"
#include <mutex>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define ATT_WAVES 4
#define ATT_STEP (ATT_WAVES * 32)  // keys a workgroup takes in one step; chunks are multiples of it
#define NEG_BIG (-1.0e30f)

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

// two floats to packed bfloat16, round to nearest even (one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

__device__ __forceinline__ f32x4 mfma16(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <int D16>
__global__ void __launch_bounds__(ATT_WAVES * 64, 2)
attn_mfma_kernel(bf16* __restrict__ out, float* __restrict__ ws_acc, float* __restrict__ ws_ml,
                 const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                 const int* __restrict__ block_tables, const int* __restrict__ seg,
                 const int* __restrict__ pos, const int* __restrict__ rows, int nh, int nkv, int page,
                 int max_blocks, int q_stride, int out_stride, float scale_log2e, int window, int nsplit, int span) {
    constexpr int D = D16 * 16;
    constexpr int KS = (D + 31) / 32;
    __shared__ float sm_acc[ATT_WAVES][D16][64][4];
    __shared__ float sm_ml[ATT_WAVES][16][2];
    const int t = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
    if (t < 0) return;   // an entry that fills up the list of a recorded step: no row (the whole workgroup leaves)
    const int G = nh / nkv;
    const int HG = (G + 15) / 16;
    const int kvh = blockIdx.y / HG, hg = blockIdx.y % HG;
    const int split = blockIdx.z;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, r = lane & 15, qg = lane >> 4;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int hcol = hg * 16 + r;
    const bool head_ok = hcol < G;
    const int head = kvh * G + (head_ok ? hcol : G - 1);

    // the chunk's valid keys [c_begin, c_end); empty: nothing to do for the whole workgroup (the
    // merge reads only the chunks between the first and the last key the token sees)
    int c_begin = split * span, c_end = c_begin + span;
    if (c_begin < lo) c_begin = lo;
    if (c_end > p + 1) c_end = p + 1;
    if (c_begin >= c_end) return;

    const int* bt = block_tables + (size_t)seg[t] * max_blocks;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    f32x4 acc[D16];
#pragma unroll
    for (int db = 0; db < D16; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = NEG_BIG, lsum = 0.f;

    // Q fragments: lane (r, qg) holds dims ks*32 + qg*8 .. +8 of head column r
    uint4 qf[KS];
    {
        const bf16* qrow = q + (size_t)t * q_stride + (size_t)head * D;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int dofs = ks * 32 + qg * 8;
            const uint4 v = *reinterpret_cast<const uint4*>(qrow + (dofs < D ? dofs : 0));
            qf[ks] = dofs < D ? v : zero4;
        }
    }
    // The chunk is walked in steps of ATT_STEP keys, 32 a wave; the loads of a step (K and V of the
    // wave's 32 keys) are issued one step ahead into a second set of registers.  They are
    // unconditional 16-byte loads from clamped addresses, masked afterwards.
    const int first_step = (c_begin - split * span) / ATT_STEP, last_step = (c_end - 1 - split * span) / ATT_STEP;
#define ATT_LOAD(KF_, VF_, STEP_)                                                                          \
    {                                                                                                      \
        const int kb_ = split * span + (STEP_) * ATT_STEP + wave * 32;                                     \
        const int kbeg_ = kb_ > c_begin ? kb_ : c_begin, kend_ = kb_ + 32 < c_end ? kb_ + 32 : c_end;     \
        if (kbeg_ < kend_) {   /* wave-uniform */                                                          \
            _Pragma("unroll") for (int tau = 0; tau < 2; ++tau) {                                          \
                /* row i of S tile tau is key kb + (i/4)*8 + tau*4 + i%4; clamped onto pages that exist */ \
                int key = kb_ + (r >> 2) * 8 + tau * 4 + (r & 3);                                          \
                key = key < kbeg_ ? kbeg_ : (key >= kend_ ? kend_ - 1 : key);                              \
                const int pg = bt[key / page];                                                             \
                const bf16* krow = kc + (((size_t)pg * nkv + kvh) * page + (key % page)) * D;              \
                _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                        \
                    const int dofs = ks * 32 + qg * 8;                                                     \
                    KF_[tau][ks] = *reinterpret_cast<const uint4*>(krow + (dofs < D ? dofs : 0));          \
                }                                                                                          \
            }                                                                                              \
            /* this lane's 8 keys of the second product are kb + qg*8 .. +8 (one page); a group with no  \
               valid key is read from the wave's first valid group instead and masked below */            \
            int key0 = kb_ + qg * 8;                                                                       \
            if (key0 >= kend_ || key0 + 8 <= kbeg_) key0 = kbeg_ & ~7;                                     \
            const int pg = bt[key0 / page];                                                                \
            const bf16* vbase = vc + ((size_t)pg * nkv + kvh) * D * page + (key0 % page);                  \
            _Pragma("unroll") for (int db = 0; db < D16; ++db)                                             \
                VF_[db] = *reinterpret_cast<const uint4*>(vbase + (size_t)(db * 16 + r) * page);           \
        }                                                                                                  \
    }
#define ATT_COMPUTE(KF_, VF_, STEP_)                                                                       \
    {                                                                                                      \
        const int kb_ = split * span + (STEP_) * ATT_STEP + wave * 32;                                     \
        const int kbeg_ = kb_ > c_begin ? kb_ : c_begin, kend_ = kb_ + 32 < c_end ? kb_ + 32 : c_end;     \
        if (kbeg_ < kend_) {   /* wave-uniform */                                                          \
            f32x4 s[2];                                                                                    \
            _Pragma("unroll") for (int tau = 0; tau < 2; ++tau) {                                          \
                s[tau] = f32x4{0.f, 0.f, 0.f, 0.f};                                                        \
                _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                        \
                    const int dofs = ks * 32 + qg * 8;                                                     \
                    s[tau] = mfma16(dofs < D ? KF_[tau][ks] : zero4, qf[ks], s[tau]);                      \
                }                                                                                          \
            }                                                                                              \
            /* lane (r, qg) holds, for head column r, keys kb + qg*8 + tau*4 + e */                       \
            float sv[8];                                                                                   \
            float mx = NEG_BIG;                                                                            \
            _Pragma("unroll") for (int tau = 0; tau < 2; ++tau)                                            \
                _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                            \
                    const int key = kb_ + qg * 8 + tau * 4 + e;                                            \
                    const bool ok = key >= kbeg_ && key < kend_;                                           \
                    const float v = ok ? s[tau][e] * scale_log2e : NEG_BIG;                                \
                    sv[tau * 4 + e] = v;                                                                   \
                    mx = fmaxf(mx, v);                                                                     \
                }                                                                                          \
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));                                                        \
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));                                                        \
            const float m_new = fmaxf(m, mx);                                                              \
            const float corr = __builtin_amdgcn_exp2f(m - m_new);                                          \
            float pe[8];                                                                                   \
            float rs = 0.f;                                                                                \
            _Pragma("unroll") for (int j = 0; j < 8; ++j) {                                                \
                pe[j] = (sv[j] > 0.5f * NEG_BIG) ? __builtin_amdgcn_exp2f(sv[j] - m_new) : 0.f;            \
                rs += pe[j];                                                                               \
            }                                                                                              \
            rs += __shfl_xor(rs, 16, 64);                                                                  \
            rs += __shfl_xor(rs, 32, 64);                                                                  \
            lsum = lsum * corr + rs;                                                                       \
            m = m_new;                                                                                     \
            uint4 pf;                                                                                      \
            pf.x = pack_bf16x2(pe[0], pe[1]);                                                              \
            pf.y = pack_bf16x2(pe[2], pe[3]);                                                              \
            pf.z = pack_bf16x2(pe[4], pe[5]);                                                              \
            pf.w = pack_bf16x2(pe[6], pe[7]);                                                              \
            const int key0 = kb_ + qg * 8;                                                                 \
            const bool vok = key0 < kend_ && key0 + 8 > kbeg_;  /* else the loaded values are another group's */ \
            _Pragma("unroll") for (int db = 0; db < D16; ++db) {                                           \
                _Pragma("unroll") for (int e = 0; e < 4; ++e) acc[db][e] *= corr;                          \
                acc[db] = mfma16(vok ? VF_[db] : zero4, pf, acc[db]);                                      \
            }                                                                                              \
        }                                                                                                  \
    }
    uint4 kfa[2][KS], vfa[D16], kfb[2][KS], vfb[D16];
    ATT_LOAD(kfa, vfa, first_step)
    for (int st = first_step; st <= last_step; st += 2) {
        if (st + 1 <= last_step) ATT_LOAD(kfb, vfb, st + 1)
        __builtin_amdgcn_sched_barrier(0);
        ATT_COMPUTE(kfa, vfa, st)
        if (st + 1 > last_step) break;
        if (st + 2 <= last_step) ATT_LOAD(kfa, vfa, st + 2)
        __builtin_amdgcn_sched_barrier(0);
        ATT_COMPUTE(kfb, vfb, st + 1)
    }
#undef ATT_LOAD
#undef ATT_COMPUTE
    // ---- merge the four waves; acc[db][e] is dim db*16 + qg*4 + e of head column r
#pragma unroll
    for (int db = 0; db < D16; ++db) *reinterpret_cast<f32x4*>(&sm_acc[wave][db][lane][0]) = acc[db];
    if (qg == 0) {
        sm_ml[wave][r][0] = m;
        sm_ml[wave][r][1] = lsum;
    }
    __syncthreads();
    float M = NEG_BIG;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; ++w) M = fmaxf(M, sm_ml[w][r][0]);
    float wgt[ATT_WAVES];
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; ++w) {
        wgt[w] = __builtin_amdgcn_exp2f(sm_ml[w][r][0] - M);
        L += sm_ml[w][r][1] * wgt[w];
    }
    if (!head_ok) return;
    const size_t slot = ((size_t)blockIdx.x * nh + head) * nsplit + split;   // the workspace is laid out by served row
    for (int db = wave; db < D16; db += ATT_WAVES) {
        f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < ATT_WAVES; ++w) {
            const f32x4 a = *reinterpret_cast<const f32x4*>(&sm_acc[w][db][lane][0]);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] += a[e] * wgt[w];
        }
        if (nsplit == 1) {
            const float inv = 1.0f / L;
            uint2 wv;
            wv.x = pack_bf16x2(o[0] * inv, o[1] * inv);
            wv.y = pack_bf16x2(o[2] * inv, o[3] * inv);
            *reinterpret_cast<uint2*>(out + (size_t)t * out_stride + (size_t)head * D + db * 16 + qg * 4) = wv;
        } else {
            *reinterpret_cast<f32x4*>(ws_acc + slot * D + db * 16 + qg * 4) = o;
        }
    }
    if (nsplit > 1 && wave == 0 && qg == 0) {
        ws_ml[slot * 2] = M;
        ws_ml[slot * 2 + 1] = L;
    }
}

// out[t, h, :] = sum_i acc_i 2^(m_i - M) / sum_i l_i 2^(m_i - M), chunks in ascending order.
// One wave per (token, head); lanes first share the chunks' (m, l), then each sums its dims.  For few
// chunks (a walk of 16 is two rounds of loads: 4.6 us against 5.5 for the kernel of four waves below).
__global__ void __launch_bounds__(64)
attn_merge_one_wave_kernel(bf16* __restrict__ out, const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
                  const int* __restrict__ pos, const int* __restrict__ rows, int nh, int D, int out_stride,
                  int window, int nsplit, int span) {
    __shared__ float wsm[64];
    const int t = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
    if (t < 0) return;   // an entry that fills up the list of a recorded step: no row (the whole workgroup leaves)
    const int h = blockIdx.y, lane = threadIdx.x;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int s_lo = lo / span, s_hi = p / span;
    const size_t base = ((size_t)blockIdx.x * nh + h) * nsplit;
    float o[4] = {0.f, 0.f, 0.f, 0.f};  // dims lane, lane+64, ... (D <= 256)
    float M = NEG_BIG, L = 0.f;
    // chunks in groups of 64: running rescale keeps one pass
    for (int g0 = s_lo; g0 <= s_hi; g0 += 64) {
        const int s = g0 + lane;
        const bool ok = s <= s_hi;
        const float ms = ok ? ws_ml[(base + s) * 2] : NEG_BIG;
        const float ls = ok ? ws_ml[(base + s) * 2 + 1] : 0.f;
        const float Mn = fmaxf(M, wave_max(ms));
        const float corr = __builtin_amdgcn_exp2f(M - Mn);
        const float w = __builtin_amdgcn_exp2f(ms - Mn);
        L = L * corr + wave_sum(ls * w);
        M = Mn;
        __syncthreads();
        wsm[lane] = w;
        __syncthreads();
        const int cnt = (s_hi - g0 + 1 < 64) ? s_hi - g0 + 1 : 64;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int dd = lane + 64 * i;
            if (dd < D) {
                float a = o[i] * corr;
                const float* src = ws_acc + (base + g0) * D + dd;
                int j = 0;
                for (; j + 8 <= cnt; j += 8) {   // eight chunks' loads in flight; the sum keeps its order
                    float v[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(j + u) * D];
#pragma unroll
                    for (int u = 0; u < 8; ++u) a += v[u] * wsm[j + u];
                }
                for (; j < cnt; ++j) a += src[(size_t)j * D] * wsm[j];
                o[i] = a;
            }
        }
    }
    const float inv = 1.0f / L;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int dd = lane + 64 * i;
        if (dd < D) out[(size_t)t * out_stride + (size_t)h * D + dd] = from_f32<bf16>(o[i] * inv);
    }
}

// out[t, h, :] = sum_i acc_i 2^(m_i - M) / sum_i l_i 2^(m_i - M) over the chunks the token sees.
// One workgroup of 4 waves per (token, head): the threads first share the chunks' (m, l) (a chunk a
// thread, at most ATT_MERGE_MAX_CHUNKS), then every wave sums a quarter of the chunks, in ascending
// order, for all dims (a lane: dims lane, lane + 64, ...; eight chunks' loads in flight), and the four
// partial sums are added in wave order.  The order of the sum depends on the number of chunks alone.
#define ATT_MERGE_WAVES 4
#define ATT_MERGE_ONE_WAVE_CHUNKS 24   // up to here the kernel of one wave is faster
#define ATT_MERGE_MAX_CHUNKS 512
__global__ void __launch_bounds__(ATT_MERGE_WAVES * 64)
attn_merge_kernel(bf16* __restrict__ out, const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
                  const int* __restrict__ pos, const int* __restrict__ rows, int nh, int D, int out_stride,
                  int window, int nsplit, int span) {
    constexpr int NT = ATT_MERGE_WAVES * 64, PER = ATT_MERGE_MAX_CHUNKS / NT;
    __shared__ float wsm[ATT_MERGE_MAX_CHUNKS];
    __shared__ float red[2][ATT_MERGE_WAVES];
    __shared__ float part[ATT_MERGE_WAVES][256];
    const int t = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
    if (t < 0) return;   // an entry that fills up the list of a recorded step: no row (the whole workgroup leaves)
    const int h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int s_lo = lo / span, s_hi = p / span, n = s_hi - s_lo + 1;
    const size_t base = ((size_t)blockIdx.x * nh + h) * nsplit + s_lo;
    float ms[PER], ls[PER];
    float mx = NEG_BIG;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = tid + NT * i;
        const bool ok = j < n;
        ms[i] = ok ? ws_ml[(base + j) * 2] : NEG_BIG;
        ls[i] = ok ? ws_ml[(base + j) * 2 + 1] : 0.f;
        mx = fmaxf(mx, ms[i]);
    }
    mx = wave_max(mx);
    if (lane == 0) red[0][wave] = mx;
    __syncthreads();
    float M = red[0][0];
#pragma unroll
    for (int w = 1; w < ATT_MERGE_WAVES; ++w) M = fmaxf(M, red[0][w]);
    float lw = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const float w = __builtin_amdgcn_exp2f(ms[i] - M);   // a chunk beyond the last: 2^(-huge) = 0
        wsm[tid + NT * i] = w;
        lw += ls[i] * w;
    }
    lw = wave_sum(lw);
    if (lane == 0) red[1][wave] = lw;
    __syncthreads();
    float L = red[1][0];
#pragma unroll
    for (int w = 1; w < ATT_MERGE_WAVES; ++w) L += red[1][w];
    // this wave's chunks [c0, c1)
    const int per_wave = (n + ATT_MERGE_WAVES - 1) / ATT_MERGE_WAVES;
    const int c0 = wave * per_wave, c1 = c0 + per_wave < n ? c0 + per_wave : n;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int dd = lane + 64 * i;
        if (dd < D) {
            float a = 0.f;
            const float* src = ws_acc + base * D + dd;
            int j = c0;
            for (; j + 8 <= c1; j += 8) {   // eight chunks' loads in flight; the sum keeps its order
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(j + u) * D];
#pragma unroll
                for (int u = 0; u < 8; ++u) a += v[u] * wsm[j + u];
            }
            for (; j < c1; ++j) a += src[(size_t)j * D] * wsm[j];
            part[wave][dd] = a;
        }
    }
    __syncthreads();
    if (tid < D) {
        float o = part[0][tid];
#pragma unroll
        for (int w = 1; w < ATT_MERGE_WAVES; ++w) o += part[w][tid];
        out[(size_t)t * out_stride + (size_t)h * D + tid] = from_f32<bf16>(o / L);
    }
}

// ------------------------------------------------------------------------------------------------
// Tiles of up to ATT_TT consecutive tokens of one request (portions of prompts): the 4 waves of a
// workgroup take 2 tokens each and share every 64-key tile of K and V through LDS (the next tile is
// already on its way: into registers, or, for heads of 128 and pages that hold whole tiles, straight
// into a second pair of LDS buffers), so a tile is read from the cache once per 8 tokens x 16 heads.  No key chunks and no
// workspace: one workgroup walks all keys its tokens see, in ascending order of absolute key
// index, 32 at a time.
// ------------------------------------------------------------------------------------------------
#define ATT_TT 8
#define ATT_NT 2
#define ATT_TK 64        // keys per tile
#define ATT_BT_LDS 2048  // block-table entries kept in LDS
#define ATT_LAZY 8.0f    // the exponent's reference point follows the maximum in steps of at least this

__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

template <int D16, bool PAGE64>
__global__ void __launch_bounds__(256, 2)
attn_tile_kernel(bf16* __restrict__ out, const bf16* __restrict__ q, const bf16* __restrict__ kc,
                 const bf16* __restrict__ vc, const int* __restrict__ block_tables, const int* __restrict__ seg,
                 const int* __restrict__ pos, const int* __restrict__ tiles, int nh, int nkv, int page,
                 int max_blocks, int q_stride, int out_stride, float scale_log2e, int window, int pair_base) {
    constexpr int D = D16 * 16;
    constexpr int KS = (D + 31) / 32;
    // K rows [key][d] and V rows [d][key] in LDS, read in 16-byte pieces by 16 rows x 4 lane groups.
    // Head size 128: rows unpadded and the pieces of a row exchanged by an exclusive-or with the row's
    // number (K: piece ^ (row & 15); V, two rows a 256-byte line: piece ^ ((row >> 1) & 7)), so the 16
    // rows one matrix operand reads fall on 16 different 16-byte bank groups whichever lanes the
    // hardware serves together.  Other head sizes: rows padded by 16 bytes.
    constexpr bool SWZ = D == 128;
    constexpr int KROW = SWZ ? D : D + 8;
    constexpr int VROW = SWZ ? ATT_TK : ATT_TK + 8;
    // DIRECT (head size 128 and pages that hold whole tiles): a tile goes from the cache into LDS without passing
    // through registers (global_load_lds_dwordx4: lane l's 16 bytes land at the instruction's LDS base + 16 l, so
    // the exchange of a row's pieces is made on the source side: the lane that fills a slot reads the piece
    // that belongs there).  The loads of the next tile are then on their way into a second pair of buffers
    // while this one is multiplied, with one barrier a tile and no stores to LDS.  Measured at 2,048 tokens: of
    // 63 us a layer, 8 were the loads into registers and 6 the stores into LDS (timing runs without them).
    constexpr bool DIRECT = SWZ && PAGE64;
    constexpr int NBUF = DIRECT ? 2 : 1;
    __shared__ __attribute__((aligned(16))) bf16 Ks2[NBUF][ATT_TK * KROW];
    __shared__ __attribute__((aligned(16))) bf16 Vs2[NBUF][D * VROW];
    const bf16* Ks = Ks2[0];   // the tile being multiplied
    const bf16* Vs = Vs2[0];
    auto k_at = [](int row, int piece) -> int { return row * KROW + (SWZ ? (piece ^ (row & 15)) : piece) * 8; };
    auto v_at = [](int row, int piece) -> int { return row * VROW + (SWZ ? (piece ^ ((row >> 1) & 7)) : piece) * 8; };
    __shared__ int bt_s[ATT_BT_LDS];
    // Items (tile, head group) in descending order of length: the longest tiles (latest positions)
    // are dispatched first.  When the whole launch is resident at once (at most two workgroups a
    // compute unit), workgroups w and w + pair_base land on the same unit (workgroups go to the
    // eight dies in turn and to a die's units in turn): the second of them then takes the items
    // from the short end, so that every unit holds a long and a short one.
    const int n_items = gridDim.x * gridDim.y;
    const int w = blockIdx.y * gridDim.x + blockIdx.x;
    const int item = (pair_base > 0 && w >= pair_base) ? n_items - 1 - (w - pair_base) : w;
    const int tile_id = gridDim.x - 1 - item / gridDim.y;
    const int by = item % gridDim.y;
    const int t0 = tiles[2 * tile_id], ntok = tiles[2 * tile_id + 1];
    if (ntok <= 0) return;   // a tile of no tokens: what fills up the list of a recorded step (the whole workgroup leaves)
    const int G = nh / nkv;
    const int HG = (G + 15) / 16;
    const int kvh = by / HG, hg = by % HG;
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, qg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: what depends on it stays in SGPRs
    const int hcol = hg * 16 + r;
    const bool head_ok = hcol < G;
    const int head = kvh * G + (head_ok ? hcol : G - 1);
    const int p_first = pos[t0], p_last = p_first + ntok - 1;
    const int lo_first = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int* bt = block_tables + (size_t)seg[t0] * max_blocks;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    // the pages of the keys this tile sees, into LDS (page lookups then cost no trip to memory)
    const int blk_first = lo_first / page, blk_count = p_last / page - blk_first + 1;
    const bool bt_in_lds = blk_count <= ATT_BT_LDS;
    if (bt_in_lds)
        for (int i = tid; i < blk_count; i += 256) bt_s[i] = bt[blk_first + i];
    auto page_of = [&](int key) -> int { return bt_in_lds ? bt_s[key / page - blk_first] : bt[key / page]; };

    // this wave's tokens
    int tok[ATT_NT], pj[ATT_NT], loj[ATT_NT];
    bool tok_ok[ATT_NT];
    uint4 qf[ATT_NT][KS];
#pragma unroll
    for (int j = 0; j < ATT_NT; ++j) {
        const int i = wave * ATT_NT + j;
        tok_ok[j] = i < ntok;
        tok[j] = t0 + (tok_ok[j] ? i : ntok - 1);
        pj[j] = p_first + (tok_ok[j] ? i : ntok - 1);
        loj[j] = (window > 0 && pj[j] - window + 1 > 0) ? pj[j] - window + 1 : 0;
        const bf16* qrow = q + (size_t)tok[j] * q_stride + (size_t)head * D;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int dofs = ks * 32 + qg * 8;
            const uint4 v = *reinterpret_cast<const uint4*>(qrow + (dofs < D ? dofs : 0));
            qf[j][ks] = dofs < D ? v : zero4;
        }
    }
    f32x4 acc[ATT_NT][D16], lacc[ATT_NT];   // lacc: every element holds the column's sum of p
    float mc[ATT_NT];                        // reference point of the exponent: (a past maximum) * scale * log2(e)
    const uint4 ones4 = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);   // bfloat16 1.0
#pragma unroll
    for (int j = 0; j < ATT_NT; ++j) {
        mc[j] = NEG_BIG;
        lacc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int db = 0; db < D16; ++db) acc[j][db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // cooperative copy of one tile of ATT_TK keys: K rows [key][d], V rows [d][key], 16-byte pieces
    constexpr int KPIECES = ATT_TK * (D / 8);
    constexpr int VPIECES = D * (ATT_TK / 8);
    constexpr int KPER = (KPIECES + 255) / 256, VPER = (VPIECES + 255) / 256;
    static_assert(KPER <= 4 && VPER <= 4, "a tile is at most four 16-byte pieces a thread");
    // PAGE64: the page size is a multiple of the tile's 64 keys, so a tile lies on one page: one page
    // lookup a tile (the same for every thread) and no clamping - keys of the page beyond the tokens'
    // reach are masked later.  Otherwise every piece finds its own page.
    // V row of piece pc: of 16 consecutive pieces the first 8 are one row and the next 8 the row 8
    // further on (not the next one): with rows 36 banks apart the two halves of a 16-lane store then
    // fall on different halves of the banks
    static_assert(ATT_TK == 64, "v_row places 8 pieces a row");
    auto v_row = [](int pc) -> int { return SWZ ? pc >> 3 : (pc >> 7) * 16 + ((pc & 127) >> 4) + 8 * ((pc >> 3) & 1); };
    int koff[4], voff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int pk = tid + i * 256 < KPIECES ? tid + i * 256 : 0;
        const int pv = tid + i * 256 < VPIECES ? tid + i * 256 : 0;
        koff[i] = (pk / (D / 8)) * D + (pk % (D / 8)) * 8;
        voff[i] = v_row(pv) * page + (pv % (ATT_TK / 8)) * 8;
    }
    const bf16* ktile = kc;
    const bf16* vtile = vc;
    auto fetch_k = [&](int kb, int i) -> uint4 {
        if (PAGE64) return *reinterpret_cast<const uint4*>(ktile + koff[i]);
        const int pc = tid + i * 256;
        const int row = (pc < KPIECES ? pc : 0) / (D / 8), col = (pc < KPIECES ? pc : 0) % (D / 8);
        int key = kb + row;
        key = key < lo_first ? lo_first : (key > p_last ? p_last : key);   // a page that exists
        const int pg = page_of(key);
        return *reinterpret_cast<const uint4*>(kc + (((size_t)pg * nkv + kvh) * page + (key % page)) * D + col * 8);
    };
    auto fetch_v = [&](int kb, int i) -> uint4 {
        if (PAGE64) return *reinterpret_cast<const uint4*>(vtile + voff[i]);
        const int pc = tid + i * 256;
        const int drow = v_row(pc < VPIECES ? pc : 0), kgrp = (pc < VPIECES ? pc : 0) % (ATT_TK / 8);
        int key0 = kb + kgrp * 8;
        if (key0 > p_last || key0 + 8 <= lo_first) key0 = lo_first & ~7;   // masked later; any valid group
        const int pg = page_of(key0);
        return *reinterpret_cast<const uint4*>(vc + (((size_t)pg * nkv + kvh) * D + drow) * page + (key0 % page));
    };
    auto stash_k = [&](int i, uint4 v) {
        const int pc = tid + i * 256;
        // Key kk of the tile lies in row (kk&32) | (kk&4)<<2 | (kk&24)>>1 | (kk&3): the 16 keys that one
        // score product's lanes read (8 consecutive keys a lane group, two products) are 16
        // consecutive rows, which the row padding spreads over all banks.
        const int kk = pc / (D / 8);
        const int prow = (kk & 32) | ((kk & 4) << 2) | ((kk & 24) >> 1) | (kk & 3);
        if (pc < KPIECES) *reinterpret_cast<uint4*>(&Ks2[0][k_at(prow, pc % (D / 8))]) = v;
    };
    auto stash_v = [&](int i, uint4 v) {
        const int pc = tid + i * 256;
        if (pc < VPIECES) *reinterpret_cast<uint4*>(&Vs2[0][v_at(v_row(pc), pc % (ATT_TK / 8))]) = v;
    };
    uint4 k0 = zero4, k1 = zero4, k2 = zero4, k3 = zero4, v0 = zero4, v1 = zero4, v2 = zero4, v3 = zero4;
    // DIRECT: instruction u of this wave fills the 64 consecutive 16-byte slots from (wave * 4 + u) * 64 on, of K and
    // of V; this lane's slot of it holds, K: piece (slot & 15) ^ (row & 15) of the key whose row it is (the inverse
    // of stash_k's row order), V: keys ((slot & 7) ^ ((row >> 1) & 7)) * 8 .. + 8 of dim row = slot >> 3
    int kdir[4], vdir[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = (wave * 4 + u) * 64 + lane;
        const int krow = i >> 4, kslot = i & 15;
        const int key = (krow & 32) | ((krow & 16) >> 2) | ((krow & 12) << 1) | (krow & 3);
        kdir[u] = key * D + ((kslot ^ (krow & 15)) * 8);
        const int vrow = i >> 3, vslot = i & 7;
        vdir[u] = vrow * page + ((vslot ^ ((vrow >> 1) & 7)) * 8);
    }
    typedef __attribute__((address_space(3))) void* lds_ptr;
#define ATT_FETCH_DIRECT(kb_, BUF_)                                                                            \
    {                                                                                                          \
        const int pg_ = page_of(kb_);                                                                          \
        const bf16* kt_ = kc + (((size_t)pg_ * nkv + kvh) * page + ((kb_) % page)) * D;                        \
        const bf16* vt_ = vc + ((size_t)pg_ * nkv + kvh) * D * page + ((kb_) % page);                          \
        _Pragma("unroll") for (int u = 0; u < 4; ++u)                                                          \
            __builtin_amdgcn_global_load_lds((const void*)(kt_ + kdir[u]), (lds_ptr)(&Ks2[BUF_][(wave * 4 + u) * 512]), 16, 0, 0); \
        _Pragma("unroll") for (int u = 0; u < 4; ++u)                                                          \
            __builtin_amdgcn_global_load_lds((const void*)(vt_ + vdir[u]), (lds_ptr)(&Vs2[BUF_][(wave * 4 + u) * 512]), 16, 0, 0); \
    }
#define ATT_FETCH(kb_)                          \
    if (PAGE64) {                               \
        const int pg_ = page_of(kb_);           \
        ktile = kc + (((size_t)pg_ * nkv + kvh) * page + ((kb_) % page)) * D; \
        vtile = vc + ((size_t)pg_ * nkv + kvh) * D * page + ((kb_) % page);   \
    }                                           \
    k0 = fetch_k(kb_, 0);                       \
    if (KPER > 1) k1 = fetch_k(kb_, 1);         \
    if (KPER > 2) k2 = fetch_k(kb_, 2);         \
    if (KPER > 3) k3 = fetch_k(kb_, 3);         \
    v0 = fetch_v(kb_, 0);                       \
    if (VPER > 1) v1 = fetch_v(kb_, 1);         \
    if (VPER > 2) v2 = fetch_v(kb_, 2);         \
    if (VPER > 3) v3 = fetch_v(kb_, 3);
#define ATT_STASH()                             \
    stash_k(0, k0);                             \
    if (KPER > 1) stash_k(1, k1);               \
    if (KPER > 2) stash_k(2, k2);               \
    if (KPER > 3) stash_k(3, k3);               \
    stash_v(0, v0);                             \
    if (VPER > 1) stash_v(1, v1);               \
    if (VPER > 2) stash_v(2, v2);               \
    if (VPER > 3) stash_v(3, v3);

    const int kb0 = lo_first & ~(ATT_TK - 1);
    __syncthreads();   // bt_s is filled
    int cur = 0;       // DIRECT: the buffers of the tile that is multiplied next
    if (DIRECT) {
        ATT_FETCH_DIRECT(kb0, 0)
    } else {
        ATT_FETCH(kb0)
    }
    // every tile begins with the exchange of the staged registers for the tile in LDS; DIRECT: with the wait
    // for this tile's loads, after which (and a barrier: everybody's have landed, and everybody is done with the
    // tile before) the loads of the next tile go into the other buffers
    auto tile_begin = [&](int kb) {
        if (DIRECT) {
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            Ks = Ks2[cur];
            Vs = Vs2[cur];
            cur ^= 1;
            if (kb + ATT_TK <= p_last) {
                if (cur) ATT_FETCH_DIRECT(kb + ATT_TK, 1) else ATT_FETCH_DIRECT(kb + ATT_TK, 0)
            }
        } else {
            __syncthreads();   // the previous tile has been consumed
            ATT_STASH()
            __syncthreads();
        }
    };
    // A tile that both tokens of the wave see whole (every tile but those on the diagonal and at a
    // window's edge) takes a path without masks, written so that matrix and vector instructions
    // alternate: a wave issues in order, so the vector work of one sub-tile has to stand between
    // the matrix instructions of another to run beside them.
    auto fast_tile = [&](int kb) {
        uint4 kf0[2][KS], kf1[2][KS];
        f32x4 s0[ATT_NT][2], s1[ATT_NT][2];
#pragma unroll
        for (int tau = 0; tau < 2; ++tau)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) kf0[tau][ks] = *reinterpret_cast<const uint4*>(&Ks[k_at(tau * 16 + r, ks * 4 + qg)]);
#pragma unroll
        for (int tau = 0; tau < 2; ++tau)
#pragma unroll
            for (int j = 0; j < ATT_NT; ++j) {
                s0[j][tau] = f32x4{0.f, 0.f, 0.f, 0.f};
                s1[j][tau] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int tau = 0; tau < 2; ++tau)
#pragma unroll
                for (int j = 0; j < ATT_NT; ++j) s0[j][tau] = mfma16(kf0[tau][ks], qf[j][ks], s0[j][tau]);
        __builtin_amdgcn_sched_barrier(0);   // the next fragments take the registers of these
#pragma unroll
        for (int tau = 0; tau < 2; ++tau)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) kf1[tau][ks] = *reinterpret_cast<const uint4*>(&Ks[k_at(32 + tau * 16 + r, ks * 4 + qg)]);
        // the reference point of the exponent follows the maximum lazily (see below); rare
#define ATT_FOLLOW(S_, PRE_)                                                                               \
        {                                                                                                  \
            /* scores become exponents relative to the reference point, in place */                       \
            float lm[ATT_NT];                                                                              \
            bool over = false;                                                                             \
            _Pragma("unroll") for (int j = 0; j < ATT_NT; ++j) {                                           \
                const bool unset = mc[j] < 0.5f * NEG_BIG;   /* no key seen yet: exponents relative to 0 */ \
                const float nm = unset ? 0.f : -mc[j];                                                     \
                _Pragma("unroll") for (int tau = 0; tau < 2; ++tau)                                        \
                    _Pragma("unroll") for (int e = 0; e < 4; ++e) S_[j][tau][e] = fmaf(S_[j][tau][e], scale_log2e, nm); \
                lm[j] = max3(max3(S_[j][0][0], S_[j][0][1], S_[j][0][2]), max3(S_[j][0][3], S_[j][1][0], S_[j][1][1]), \
                             fmaxf(S_[j][1][2], S_[j][1][3]));                                             \
                over = over || unset || lm[j] > ATT_LAZY;                                                  \
            }                                                                                              \
            if (__builtin_amdgcn_ballot_w64(over) != 0ull) {                                               \
                PRE_                                                                                       \
                _Pragma("unroll") for (int j = 0; j < ATT_NT; ++j) {                                       \
                    float mx = lm[j];                                                                      \
                    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));                                                \
                    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));                                                \
                    const bool unset = mc[j] < 0.5f * NEG_BIG;                                             \
                    const bool up = unset || mx > ATT_LAZY;   /* the same in the four lanes of a column */ \
                    const float shift = up ? mx : 0.f;                                                     \
                    const float corr = unset ? 1.0f : __builtin_amdgcn_exp2f(-shift);   /* unset: sums are 0 */ \
                    mc[j] = unset ? mx : mc[j] + shift;                                                    \
                    _Pragma("unroll") for (int tau = 0; tau < 2; ++tau)                                    \
                        _Pragma("unroll") for (int e = 0; e < 4; ++e) S_[j][tau][e] -= shift;              \
                    _Pragma("unroll") for (int e = 0; e < 4; ++e) lacc[j][e] *= corr;                      \
                    _Pragma("unroll") for (int db = 0; db < D16; ++db)                                     \
                        _Pragma("unroll") for (int e = 0; e < 4; ++e) acc[j][db][e] *= corr;               \
                }                                                                                          \
            }                                                                                              \
        }
        // one quarter of a sub-tile's p: token J_, key tile TAU_ -> two words of its fragment
#define ATT_PQ(S_, J_, TAU_, LO_, HI_)                                                                     \
        {                                                                                                  \
            const float p0 = __builtin_amdgcn_exp2f(S_[J_][TAU_][0]);                                      \
            const float p1 = __builtin_amdgcn_exp2f(S_[J_][TAU_][1]);                                      \
            const float p2 = __builtin_amdgcn_exp2f(S_[J_][TAU_][2]);                                      \
            const float p3 = __builtin_amdgcn_exp2f(S_[J_][TAU_][3]);                                      \
            LO_ = pack_bf16x2(p0, p1);                                                                     \
            HI_ = pack_bf16x2(p2, p3);                                                                     \
        }
        ATT_FOLLOW(s0, )
        // scores of the second sub-tile on the matrix cores, p of the first on the vector units
        uint4 pf0[ATT_NT], pf1[ATT_NT];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int tau = 0; tau < 2; ++tau)
#pragma unroll
                for (int j = 0; j < ATT_NT; ++j) s1[j][tau] = mfma16(kf1[tau][ks], qf[j][ks], s1[j][tau]);
            if (ks == 0) ATT_PQ(s0, 0, 0, pf0[0].x, pf0[0].y)
            if (ks == 1 || KS == 1) ATT_PQ(s0, 0, 1, pf0[0].z, pf0[0].w)
            if (ks == 2 || (KS <= 2 && ks == KS - 1)) ATT_PQ(s0, 1, 0, pf0[1].x, pf0[1].y)
            if (ks == KS - 1) ATT_PQ(s0, 1, 1, pf0[1].z, pf0[1].w)
            __builtin_amdgcn_sched_barrier(0);
        }
        // the next tile leaves for the registers only now: until here they held score fragments
        if (!DIRECT && kb + ATT_TK <= p_last) { ATT_FETCH(kb + ATT_TK) }
        // values of the first sub-tile; their products stand between the p of the second
        // (should the reference point move now, the first sub-tile's products, made with the old one,
        // are added first, and the interleaved block below adds zeros in their place)
        ATT_FOLLOW(s1, {
            _Pragma("unroll") for (int j = 0; j < ATT_NT; ++j) lacc[j] = mfma16(ones4, pf0[j], lacc[j]);
            _Pragma("unroll") for (int db = 0; db < D16; ++db) {
                const uint4 v = *reinterpret_cast<const uint4*>(&Vs[v_at(db * 16 + r, qg)]);
                _Pragma("unroll") for (int j = 0; j < ATT_NT; ++j) acc[j][db] = mfma16(v, pf0[j], acc[j][db]);
            }
            _Pragma("unroll") for (int j = 0; j < ATT_NT; ++j) pf0[j] = zero4;
        })
        constexpr int DH = (D16 + 1) / 2;   // value fragments in two halves: fewer registers live
        uint4 vf[DH];
#pragma unroll
        for (int db = 0; db < DH; ++db) vf[db] = *reinterpret_cast<const uint4*>(&Vs[v_at(db * 16 + r, qg)]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < ATT_NT; ++j) lacc[j] = mfma16(ones4, pf0[j], lacc[j]);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < DH; ++i) {
                const int db = h * DH + i;
                if (db < D16) {
#pragma unroll
                    for (int j = 0; j < ATT_NT; ++j) acc[j][db] = mfma16(vf[i], pf0[j], acc[j][db]);
                }
                if (h == 0 && i == 0) ATT_PQ(s1, 0, 0, pf1[0].x, pf1[0].y)
                if (h == 0 && i == DH - 1) ATT_PQ(s1, 0, 1, pf1[0].z, pf1[0].w)
                if (h == 1 && i == 0) ATT_PQ(s1, 1, 0, pf1[1].x, pf1[1].y)
                if (h == 1 && i == DH - 1) ATT_PQ(s1, 1, 1, pf1[1].z, pf1[1].w)
                __builtin_amdgcn_sched_barrier(0);
            }
            // the next half: second half of this sub-tile, then the first of the other
#pragma unroll
            for (int i = 0; i < DH; ++i) {
                const int db = (h == 0 ? DH : 0) + i;
                if (db < D16) vf[i] = *reinterpret_cast<const uint4*>(&Vs[v_at(db * 16 + r, (h == 0 ? 0 : 4) + qg)]);
            }
        }
#pragma unroll
        for (int j = 0; j < ATT_NT; ++j) lacc[j] = mfma16(ones4, pf1[j], lacc[j]);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < DH; ++i) {
                const int db = h * DH + i;
                if (db < D16) {
#pragma unroll
                    for (int j = 0; j < ATT_NT; ++j) acc[j][db] = mfma16(vf[i], pf1[j], acc[j][db]);
                }
            }
            if (h == 0) {
#pragma unroll
                for (int i = 0; i < DH; ++i) {
                    const int db = DH + i;
                    if (db < D16) vf[i] = *reinterpret_cast<const uint4*>(&Vs[v_at(db * 16 + r, 4 + qg)]);
                }
            }
        }
#undef ATT_FOLLOW
#undef ATT_PQ
    };
    // any tile: masks where a token does not see a key
    auto general_tile = [&](int kb) {
        if (!DIRECT && kb + ATT_TK <= p_last) { ATT_FETCH(kb + ATT_TK) }   // in flight while this tile is multiplied
        // The score products of both 32-key sub-tiles are issued first, so that the matrix cores
        // work on the second while the vector units do the softmax of the first.
        constexpr int NSUB = ATT_TK / 32;
        bool any[NSUB];
        f32x4 s[NSUB][ATT_NT][2];
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub) {
            const int kbs = kb + sub * 32;
            any[sub] = kbs <= pj[ATT_NT - 1] && kbs + 32 > loj[0];   // wave-uniform
            if (!any[sub]) continue;
            uint4 kf[2][KS];
#pragma unroll
            for (int tau = 0; tau < 2; ++tau) {
                const int row = sub * 32 + tau * 16 + r;   // = key sub*32 + (r>>2)*8 + tau*4 + (r&3)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int dofs = ks * 32 + qg * 8;
                    kf[tau][ks] = (D % 32 == 0 || dofs < D)
                                      ? *reinterpret_cast<const uint4*>(&Ks[k_at(row, (D % 32 == 0 ? dofs : (dofs < D ? dofs : 0)) / 8)])
                                      : zero4;
                }
#pragma unroll
                for (int j = 0; j < ATT_NT; ++j) s[sub][j][tau] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            // four independent accumulator chains (2 key tiles x 2 tokens), interleaved over d
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int tau = 0; tau < 2; ++tau)
#pragma unroll
                    for (int j = 0; j < ATT_NT; ++j) s[sub][j][tau] = mfma16(kf[tau][ks], qf[j][ks], s[sub][j][tau]);
        }
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub) {
            if (!any[sub]) continue;
            const int kbs = kb + sub * 32;
            // Softmax on raw scores, the scale inside the exponent's multiply-add.  The reference
            // point mc (in units of the exponent) is not the running maximum itself: it is raised
            // to a column's maximum only when that exceeds it by more than ATT_LAZY, so p <= 2^ATT_LAZY
            // and on most sub-tiles no lane talks to another.  The row sums come out of the matrix
            // cores with the values (a row of ones), from the same rounded p.  Sub-tiles that every
            // token of the wave sees whole (all but the diagonal and a window's edge) skip the masks.
            const bool full = kbs + 31 <= pj[0] && kbs >= loj[ATT_NT - 1];   // wave-uniform
            float sv[ATT_NT][8], lm[ATT_NT];
            bool over = false;
#pragma unroll
            for (int j = 0; j < ATT_NT; ++j) {
#pragma unroll
                for (int tau = 0; tau < 2; ++tau)
#pragma unroll
                    for (int e = 0; e < 4; ++e) sv[j][tau * 4 + e] = s[sub][j][tau][e];
                if (!full) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int key = kbs + qg * 8 + i;
                        sv[j][i] = (key >= loj[j] && key <= pj[j]) ? sv[j][i] : NEG_BIG;
                    }
                }
                lm[j] = max3(max3(sv[j][0], sv[j][1], sv[j][2]), max3(sv[j][3], sv[j][4], sv[j][5]), max3(sv[j][6], sv[j][7], sv[j][7]));
                // (a column whose keys are all masked here leaves the reference point alone: it stays
                // unset, which the mask-free path tests by its size)
                over = over || (lm[j] > 0.5f * NEG_BIG && fmaf(lm[j], scale_log2e, -mc[j]) > ATT_LAZY);
            }
            if (__builtin_amdgcn_ballot_w64(over) != 0ull) {
#pragma unroll
                for (int j = 0; j < ATT_NT; ++j) {
                    float mx = lm[j];
                    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                    const float mxc = mx * scale_log2e;
                    const bool up = mx > 0.5f * NEG_BIG && mxc - mc[j] > ATT_LAZY;   // the same in the four lanes of a column
                    const float corr = up ? __builtin_amdgcn_exp2f(mc[j] - mxc) : 1.0f;
                    mc[j] = up ? mxc : mc[j];
#pragma unroll
                    for (int e = 0; e < 4; ++e) lacc[j][e] *= corr;
#pragma unroll
                    for (int db = 0; db < D16; ++db)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[j][db][e] *= corr;
                }
            }
            uint4 pf[ATT_NT];
#pragma unroll
            for (int j = 0; j < ATT_NT; ++j) {
                float pe[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) pe[i] = __builtin_amdgcn_exp2f(fmaf(sv[j][i], scale_log2e, -mc[j]));
                if (!full) {   // a masked score of a row that has seen no key yet would give 2^0
#pragma unroll
                    for (int i = 0; i < 8; ++i) pe[i] = (sv[j][i] > 0.5f * NEG_BIG) ? pe[i] : 0.f;
                }
                pf[j].x = pack_bf16x2(pe[0], pe[1]);
                pf[j].y = pack_bf16x2(pe[2], pe[3]);
                pf[j].z = pack_bf16x2(pe[4], pe[5]);
                pf[j].w = pack_bf16x2(pe[6], pe[7]);
                lacc[j] = mfma16(ones4, pf[j], lacc[j]);
            }
            const int key0 = kbs + qg * 8;
            const bool vok = key0 <= p_last && key0 + 8 > lo_first;   // else the tile holds another group's values
#pragma unroll
            for (int db = 0; db < D16; ++db) {
                const uint4 v = *reinterpret_cast<const uint4*>(&Vs[v_at(db * 16 + r, sub * 4 + qg)]);
                const uint4 vf = (PAGE64 || vok) ? v : zero4;   // PAGE64: the tile's own page, finite, times p = 0
#pragma unroll
                for (int j = 0; j < ATT_NT; ++j) acc[j][db] = mfma16(vf, pf[j], acc[j][db]);
            }
        }
    };
    // Tiles [kb_a, kb_b) are seen whole by every token of the workgroup: from the window's edge of the
    // last token (the start without a window) to the tile before the first token's own.  Three loops
    // rather than one with a branch: each keeps its own registers.
    const int lo_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
    int kb_a = (lo_last + ATT_TK - 1) & ~(ATT_TK - 1);
    int kb_b = ((p_first + 1) / ATT_TK) * ATT_TK;
    if (D % 32 != 0 || kb_b < kb_a) kb_a = kb_b = kb0;
    int kb = kb0;
    for (; kb < kb_a && kb <= p_last; kb += ATT_TK) {
        tile_begin(kb);
        general_tile(kb);
    }
    for (; kb < kb_b; kb += ATT_TK) {
        tile_begin(kb);
        fast_tile(kb);
    }
    for (; kb <= p_last; kb += ATT_TK) {
        tile_begin(kb);
        general_tile(kb);
    }
    if (!head_ok) return;
#pragma unroll
    for (int j = 0; j < ATT_NT; ++j) {
        if (!tok_ok[j]) continue;
        const float inv = 1.0f / lacc[j][0];
        bf16* orow = out + (size_t)tok[j] * out_stride + (size_t)head * D;
#pragma unroll
        for (int db = 0; db < D16; ++db) {
            uint2 w;
            w.x = pack_bf16x2(acc[j][db][0] * inv, acc[j][db][1] * inv);
            w.y = pack_bf16x2(acc[j][db][2] * inv, acc[j][db][3] * inv);
            *reinterpret_cast<uint2*>(orow + db * 16 + qg * 4) = w;
        }
    }
}

#undef ATT_FETCH
#undef ATT_FETCH_DIRECT
#undef ATT_STASH

extern "C" int ilm_attn_tile_tokens() { return ATT_TT; }

extern "C" int ilm_attn_tile(void* out, const void* q, const void* kc, const void* vc, const void* block_tables,
                             const void* seg, const void* pos, const void* tiles, int n_tiles, int nh, int nkv,
                             int d, int page, int max_blocks, int q_stride, int out_stride, float scale,
                             int window, hipStream_t stream) {
    ILM_REQUIRE(n_tiles > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn_tile: bad sizes");
    ILM_REQUIRE(d % 16 == 0 && d >= 16 && d <= 128, "attn_tile: head size %d is not a multiple of 16 up to 128", d);
    ILM_REQUIRE(page % 16 == 0 && page > 0, "attn_tile: page size %d is not a multiple of 16", page);
    ILM_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0 && ((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 7) == 0,
                "attn_tile: q and out rows must be 16-byte / 8-byte aligned");
    const int G = nh / nkv, HG = (G + 15) / 16;
    ILM_REQUIRE(nkv * HG <= 65535, "attn_tile: grid too large");
    dim3 grid(n_tiles, nkv * HG);
    const float sl2 = scale * 1.4426950408889634f;
    const int cus = ilm_num_cus();
    const long long n_items = (long long)n_tiles * nkv * HG;
    const int pair_base = (n_items > cus && n_items <= 2 * cus) ? cus : 0;
#define AT_ARGS (bf16*)out, (const bf16*)q, (const bf16*)kc, (const bf16*)vc, (const int*)block_tables, (const int*)seg, \
                (const int*)pos, (const int*)tiles, nh, nkv, page, max_blocks, q_stride, out_stride, sl2, window, pair_base
#define AT_CASE(D16)                                                                   \
    case D16:                                                                          \
        if (page % ATT_TK == 0) attn_tile_kernel<D16, true><<<grid, 256, 0, stream>>>(AT_ARGS);  \
        else attn_tile_kernel<D16, false><<<grid, 256, 0, stream>>>(AT_ARGS);          \
        break
    switch (d / 16) {
        AT_CASE(1); AT_CASE(2); AT_CASE(3); AT_CASE(4); AT_CASE(5); AT_CASE(6); AT_CASE(7); AT_CASE(8);
        default: ILM_REQUIRE(false, "attn_tile: head size %d", d);
    }
#undef AT_CASE
#undef AT_ARGS
    ILM_LAUNCH_CHECK("attn_tile");
    return 0;
}


extern "C" int ilm_attn_mfma_step() { return ATT_STEP; }

static int attn_mfma_launch(void* out, void* ws_acc, void* ws_ml, const void* q, const void* kc,
                            const void* vc, const void* block_tables, const void* seg, const void* pos,
                            const void* rows, int T_, int nh, int nkv, int d, int page, int max_blocks,
                            int q_stride, int out_stride, float scale, int window, int nsplit, int span,
                            hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn_mfma: bad head counts nh=%d nkv=%d", nh, nkv);
    ILM_REQUIRE(d % 16 == 0 && d >= 16 && d <= 128, "attn_mfma: head size %d is not a multiple of 16 up to 128", d);
    ILM_REQUIRE(page % 16 == 0 && page > 0, "attn_mfma: page size %d is not a multiple of 16", page);
    ILM_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0 && ((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 7) == 0,
                "attn_mfma: q and out rows must be 16-byte / 8-byte aligned");
    ILM_REQUIRE(nsplit >= 1 && (nsplit == 1 || (ws_acc != nullptr && ws_ml != nullptr)), "attn_mfma: workspace missing");
    ILM_REQUIRE(span > 0 && span % ATT_STEP == 0, "attn_mfma: chunk of %d keys is no multiple of %d", span, ATT_STEP);
    const int G = nh / nkv, HG = (G + 15) / 16;
    ILM_REQUIRE(nkv * HG <= 65535 && nsplit <= ATT_MERGE_MAX_CHUNKS, "attn_mfma: at most %d chunks, got %d", ATT_MERGE_MAX_CHUNKS, nsplit);
    dim3 grid(T_, nkv * HG, nsplit);
    const float sl2 = scale * 1.4426950408889634f;
#define AM_CASE(D16)                                                                                           \
    case D16:                                                                                                  \
        attn_mfma_kernel<D16><<<grid, ATT_WAVES * 64, 0, stream>>>(                                            \
            (bf16*)out, (float*)ws_acc, (float*)ws_ml, (const bf16*)q, (const bf16*)kc, (const bf16*)vc,      \
            (const int*)block_tables, (const int*)seg, (const int*)pos, (const int*)rows, nh, nkv, page,      \
            max_blocks, q_stride, out_stride, sl2, window, nsplit, span);                                      \
        break
    switch (d / 16) {
        AM_CASE(1); AM_CASE(2); AM_CASE(3); AM_CASE(4); AM_CASE(5); AM_CASE(6); AM_CASE(7); AM_CASE(8);
        default: ILM_REQUIRE(false, "attn_mfma: head size %d", d);
    }
#undef AM_CASE
    ILM_LAUNCH_CHECK("attn_mfma");
    if (nsplit > 1) {
        dim3 g2(T_, nh);
        if (nsplit <= ATT_MERGE_ONE_WAVE_CHUNKS)
            attn_merge_one_wave_kernel<<<g2, 64, 0, stream>>>((bf16*)out, (const float*)ws_acc, (const float*)ws_ml, (const int*)pos,
                                                              (const int*)rows, nh, d, out_stride, window, nsplit, span);
        else
            attn_merge_kernel<<<g2, ATT_MERGE_WAVES * 64, 0, stream>>>((bf16*)out, (const float*)ws_acc, (const float*)ws_ml,
                                                                       (const int*)pos, (const int*)rows, nh, d, out_stride,
                                                                       window, nsplit, span);
        ILM_LAUNCH_CHECK("attn_merge");
    }
    return 0;
}

extern "C" int ilm_attn_mfma(void* out, void* ws_acc, void* ws_ml, const void* q, const void* kc,
                             const void* vc, const void* block_tables, const void* seg, const void* pos,
                             const void* rows, int T_, int nh, int nkv, int d, int page, int max_blocks,
                             int q_stride, int out_stride, float scale, int window, int nsplit, int span,
                             hipStream_t stream) {
    return attn_mfma_launch(out, ws_acc, ws_ml, q, kc, vc, block_tables, seg, pos, rows, T_, nh, nkv, d, page, max_blocks,
                            q_stride, out_stride, scale, window, nsplit, span, stream);
}

// ------------------------------------------------------------------------------------------------
// The same attention for callers that cannot allocate (see no_alloc.h): the chunks' partial results
// go to a file-scope device array instead of a workspace the caller brings.
// ------------------------------------------------------------------------------------------------
static __device__ __align__(256) float scratch[ILM_ATTN_SCRATCH_FLOATS];

// The array's device address, per device: each GPU holds its own copy at its own address.  In host
// code the array's name is only a stand-in for the symbol; what kernels get is the pointer looked
// up here, once per device, with that device current.
#define ILM_MAX_DEVICES 64
static float* scratch_ptr[ILM_MAX_DEVICES];
static std::mutex scratch_mutex;

static int scratch_of_current_device(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    ILM_REQUIRE(e == hipSuccess && dev >= 0 && dev < ILM_MAX_DEVICES, "attn_mfma_static: no current device (%s)",
                hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        ILM_REQUIRE(e == hipSuccess && p != nullptr, "attn_mfma_static: the scratch array has no address on device %d (%s)",
                    dev, hipGetErrorString(e));
        scratch_ptr[dev] = p;
    }
    *ptr = scratch_ptr[dev];
    return 0;
}

extern "C" long ilm_attn_static_scratch_floats() { return (long)ILM_ATTN_SCRATCH_FLOATS; }

extern "C" int ilm_attn_static_init() {
    float* base = nullptr;
    return scratch_of_current_device(&base);
}

extern "C" int ilm_attn_mfma_static(void* out, const void* q, const void* kc, const void* vc,
                                    const void* block_tables, const void* seg, const void* pos, const void* rows,
                                    int T_, int nh, int nkv, int d, int page, int max_blocks, int q_stride,
                                    int out_stride, float scale, int window, int nsplit, int span,
                                    hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && d > 0 && nsplit >= 1, "attn_mfma_static: bad sizes T=%d nh=%d d=%d chunks=%d", T_, nh, d, nsplit);
    float* ws_acc = nullptr;
    float* ws_ml = nullptr;
    if (nsplit > 1) {
        const long long acc_floats = (long long)T_ * nh * nsplit * d, ml_floats = (long long)T_ * nh * nsplit * 2;
        ILM_REQUIRE(acc_floats + ml_floats <= (long long)ILM_ATTN_SCRATCH_FLOATS,
                    "attn_mfma_static: %d tokens x %d heads x %d chunks x (%d + 2) floats = %lld exceed the static "
                    "scratch of %lld floats; use fewer chunks or tokens a call, or ilm_attn_mfma with a workspace",
                    T_, nh, nsplit, d, acc_floats + ml_floats, (long long)ILM_ATTN_SCRATCH_FLOATS);
        float* base = nullptr;
        if (scratch_of_current_device(&base) != 0) return -1;
        ws_acc = base;
        ws_ml = base + acc_floats;   // d is a multiple of 16: 64-byte aligned
    }
    return attn_mfma_launch(out, ws_acc, ws_ml, q, kc, vc, block_tables, seg, pos, rows, T_, nh, nkv, d, page, max_blocks,
                            q_stride, out_stride, scale, window, nsplit, span, stream);
}
