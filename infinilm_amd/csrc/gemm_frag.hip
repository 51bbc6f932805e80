// Products of up to 64 rows of X with W streamed once, both operands in fragment order (frag.h), every
// output with one owner: the projections of a decode step in bfloat16.
//
// A workgroup of 8 waves takes NT tiles of 16 rows of W and all rows of X.  The waves split the workgroup's
// range of K evenly; a wave has the W fragments of up to ROUND k-steps in flight at once (a fragment is 1 KB
// of consecutive bytes: W comes in at the memory's speed) and streams the X fragments of XC steps beside
// them, a chunk ahead (X is read by every workgroup, from the L2s, also 1 KB an instruction).  The waves'
// partial tiles meet in LDS and are summed in wave order: the order of a sum depends on K alone, not on the
// number of rows or on the batch.  The thread that reduces an output applies the epilogue:
//
//   plain    C = alpha (X W^T + bias): bfloat16 or float rows, float parts of a K split over blockIdx.y (summed
//            by the next add+RMSNorm), or bfloat16 in fragment order for the next product
//   swiglu   tiles come in pairs (gate rows, up rows of the same 16 outputs): act = silu(gate) * up in fragment
//            order for the down projection; with the partial sums of squares that the tail epilogue left, the
//            rows are first divided by their root mean square (the norm before the feed-forward, finished here)
//   rope     tiles come in pairs (first and second rows of 16 rotation pairs of a q, k or v head): q rotated into
//            plain rows for the attention, k rotated and v into the paged cache
//   tail     r += alpha (X W^T + bias) into the float residual stream in place, xw = bfloat16(r * w) in fragment
//            order with the following norm's weight, and per tile the rows' partial sums of squares
#include "common.h"
#include "frag.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define GF_WAVES 8
#define GF_SS_ROWS 64    // rows of a tile's record of partial sums of squares

enum { GF_PLAIN = 0, GF_SWIGLU = 1, GF_ROPE = 2, GF_TAIL = 3 };
enum { GF_OUT_BF16 = 0, GF_OUT_F32 = 1, GF_OUT_FRAG = 2 };

struct GfArgs {
    const uint4* Wf;
    const uint4* Xf;
    const bf16* bias;
    int M, N, ksteps, steps_per_part, units;
    float alpha;
    // plain
    void* C;
    int ldc, out_kind;
    long part_stride;
    // swiglu (N = I outputs) and tail: fragment-order result, partial sums of squares
    uint4* out_frag;
    const float* ss_in;   // swiglu: [ss_tiles][GF_SS_ROWS] from a tail epilogue, or null
    int ss_tiles, norm_width;
    float eps;
    // rope
    bf16* Q;
    int ldq;
    const int* pos;
    const float* cosT;
    const float* sinT;
    bf16* kc;
    bf16* vc;
    const int* slots;
    int nh, nkv, d, page;
    // tail
    float* R;
    int ldr;
    const void* norm_w;
    int norm_w_f32;
    float* ss_out;
};

__device__ __forceinline__ f32x4 gf_mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ float gf_round(float v) { return to_f32(from_f32<bf16>(v)); }

template <int MG, int NT, int ROUND, int EPI>
__global__ void __launch_bounds__(GF_WAVES * 64)
gemm_frag_kernel(const GfArgs A) {
    __shared__ __align__(16) float part[NT][MG][GF_WAVES][64][4];
    __shared__ __align__(16) float ssr[GF_WAVES][GF_SS_ROWS];
    // the wave's number as a scalar: every index of a k-step is then one too, and a load's address a scalar base
    // plus the lane's offset (as a per-lane value it costs registers for every load, and those run out: the
    // compiler then parks fragments in scratch memory, which waits for all loads in flight)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int unit = blockIdx.x;
    constexpr int XC = MG <= 2 ? 4 : 2;   // k-steps a chunk of X fragments (two chunks in flight)
    // ---- the wave's k-steps
    const int p0s = blockIdx.y * A.steps_per_part;
    const int p1s = p0s + A.steps_per_part < A.ksteps ? p0s + A.steps_per_part : A.ksteps;
    const int per = (p1s - p0s + GF_WAVES - 1) / GF_WAVES;
    const int s_begin = p0s + wave * per;
    const int s_end = s_begin + per < p1s ? s_begin + per : p1s;

    // swiglu after a tail epilogue: the rows' sums of squares, four rows a thread, gathered while W arrives
    float4 ss_sum = make_float4(0.f, 0.f, 0.f, 0.f);
    constexpr int SSQ = GF_SS_ROWS / 4, SSC = GF_WAVES * 64 / SSQ;   // all 64 rows of a record, whatever M (rows beyond M are not used)
    if (EPI == GF_SWIGLU && A.ss_in != nullptr) {
        const float4* sp = reinterpret_cast<const float4*>(A.ss_in) + threadIdx.x % SSQ;
        int tl = threadIdx.x / SSQ;
        for (; tl + 3 * SSC < A.ss_tiles; tl += 4 * SSC) {
            const float4 v0 = sp[(size_t)tl * (GF_SS_ROWS / 4)], v1 = sp[(size_t)(tl + SSC) * (GF_SS_ROWS / 4)];
            const float4 v2 = sp[(size_t)(tl + 2 * SSC) * (GF_SS_ROWS / 4)], v3 = sp[(size_t)(tl + 3 * SSC) * (GF_SS_ROWS / 4)];
            ss_sum.x += (v0.x + v1.x) + (v2.x + v3.x);
            ss_sum.y += (v0.y + v1.y) + (v2.y + v3.y);
            ss_sum.z += (v0.z + v1.z) + (v2.z + v3.z);
            ss_sum.w += (v0.w + v1.w) + (v2.w + v3.w);
        }
        for (; tl < A.ss_tiles; tl += SSC) {
            const float4 v0 = sp[(size_t)tl * (GF_SS_ROWS / 4)];
            ss_sum.x += v0.x; ss_sum.y += v0.y; ss_sum.z += v0.z; ss_sum.w += v0.w;
        }
    }

    f32x4 acc[NT][MG];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[t][g] = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    for (int s0 = s_begin; s0 < s_end; s0 += ROUND) {
        // unconditional loads from clamped steps; what lies beyond the wave's range is replaced by zeros on the X side
        uint4 a[ROUND][NT];
#pragma unroll
        for (int u = 0; u < ROUND; ++u) {
            const int s = s0 + u < s_end ? s0 + u : s_end - 1;
#pragma unroll
            for (int t = 0; t < NT; ++t) a[u][t] = A.Wf[((size_t)(unit * NT + t) * A.ksteps + s) * 64 + lane];
        }
        uint4 b[2][XC][MG];
#define GF_LOADX(BUF_, U_)                                                                       \
        _Pragma("unroll") for (int u = 0; u < XC; ++u) {                                      \
            const int s = s0 + (U_) + u < s_end ? s0 + (U_) + u : s_end - 1;                     \
            _Pragma("unroll") for (int g = 0; g < MG; ++g) b[BUF_][u][g] = A.Xf[((size_t)s * MG + g) * 64 + lane]; \
        }
#define GF_MULX(BUF_, U_)                                                                        \
        _Pragma("unroll") for (int u = 0; u < XC; ++u) {                                      \
            const bool ok = s0 + (U_) + u < s_end;                                               \
            _Pragma("unroll") for (int g = 0; g < MG; ++g) {                                     \
                const uint4 xv = ok ? b[BUF_][u][g] : zero;                                      \
                _Pragma("unroll") for (int t = 0; t < NT; ++t) acc[t][g] = gf_mfma(a[(U_) + u][t], xv, acc[t][g]); \
            }                                                                                    \
        }
        GF_LOADX(0, 0)
#pragma unroll
        for (int uu = 0; uu < ROUND; uu += 2 * XC) {   // (not `u`: the macros' own loops use that name)
            if (uu + XC < ROUND) GF_LOADX(1, uu + XC)
            __builtin_amdgcn_sched_barrier(0);
            GF_MULX(0, uu)
            __builtin_amdgcn_sched_barrier(0);
            if (uu + 2 * XC < ROUND) GF_LOADX(0, uu + 2 * XC)
            __builtin_amdgcn_sched_barrier(0);
            if (uu + XC < ROUND) GF_MULX(1, uu + XC)
            __builtin_amdgcn_sched_barrier(0);
        }
#undef GF_LOADX
#undef GF_MULX
    }
    // acc[t][g][e] of lane (r, q): row 4 q + e of tile t, row 16 g + r of X
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int g = 0; g < MG; ++g) *reinterpret_cast<f32x4*>(&part[t][g][wave][lane][0]) = acc[t][g];
    if (EPI == GF_SWIGLU && A.ss_in != nullptr) {
#pragma unroll
        for (int o = SSQ; o < 64; o <<= 1) {
            ss_sum.x += __shfl_xor(ss_sum.x, o, 64);
            ss_sum.y += __shfl_xor(ss_sum.y, o, 64);
            ss_sum.z += __shfl_xor(ss_sum.z, o, 64);
            ss_sum.w += __shfl_xor(ss_sum.w, o, 64);
        }
        if (lane < SSQ) *reinterpret_cast<float4*>(&ssr[wave][lane * 4]) = ss_sum;
    }
    __syncthreads();

    // ---- epilogue: an item is (tile or pair of tiles, group g, row m16 of the group, quarter qq of the tile's rows);
    // its thread sums the four outputs e of lane qq * 16 + m16 over the waves
    auto reduce4 = [&](int t, int g, int l) -> f32x4 {
        f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < GF_WAVES; ++w) v += *reinterpret_cast<const f32x4*>(&part[t][g][w][l][0]);
        return v;
    };
    constexpr int SETS = (EPI == GF_SWIGLU || EPI == GF_ROPE) ? NT / 2 : NT;   // tiles or pairs of tiles a workgroup
    for (int it = threadIdx.x; it < SETS * MG * 64; it += GF_WAVES * 64) {
        const int qq = it & 3, m16 = (it >> 2) & 15, sg = it >> 6;
        const int set = sg / MG, g = sg % MG;
        const int l = qq * 16 + m16, m = 16 * g + m16;
        if (EPI == GF_PLAIN) {
            const int n = (unit * NT + set) * 16 + 4 * qq;
            if (m >= A.M || n >= A.N) continue;
            f32x4 v = reduce4(set, g, l);
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x = v[e];
                if (A.bias != nullptr && blockIdx.y == 0 && n + e < A.N) x += to_f32(A.bias[n + e]);
                o[e] = A.alpha * x;
            }
            if (A.out_kind == GF_OUT_F32) {
                float* dst = reinterpret_cast<float*>(A.C) + (size_t)blockIdx.y * A.part_stride + (size_t)m * A.ldc + n;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < A.N) dst[e] = o[e];
            } else if (A.out_kind == GF_OUT_BF16) {
                bf16* dst = reinterpret_cast<bf16*>(A.C) + (size_t)m * A.ldc + n;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < A.N) dst[e] = from_f32<bf16>(o[e]);
            } else {
                bf16 ob[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) ob[e] = from_f32<bf16>(n + e < A.N ? o[e] : 0.f);
                bf16* dst = reinterpret_cast<bf16*>(A.out_frag + frag_x_chunk(m, n >> 3, MG)) + (n & 7);
                *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(ob);
            }
        } else if (EPI == GF_SWIGLU) {
            const int i0 = (unit * (NT / 2) + set) * 16 + 4 * qq;   // the item's four outputs of the feed-forward's width
            if (m >= A.M) continue;
            float rstd = 1.0f;
            if (A.ss_in != nullptr) {
                float tot = 0.f;
#pragma unroll
                for (int w = 0; w < GF_WAVES; ++w) tot += ssr[w][m];
                rstd = 1.0f / sqrtf(tot / (float)A.norm_width + A.eps);
            }
            const f32x4 vg = reduce4(2 * set, g, l), vu = reduce4(2 * set + 1, g, l);
            bf16 ob[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float a = vg[e] * rstd, b = vu[e] * rstd;
                if (A.bias != nullptr && i0 + e < A.N) {
                    a += to_f32(A.bias[i0 + e]);
                    b += to_f32(A.bias[A.N + i0 + e]);
                }
                a = gf_round(a);   // gate and up rounded to bfloat16 before the activation, as the unfused path stores them
                b = gf_round(b);
                ob[e] = from_f32<bf16>(i0 + e < A.N ? a / (1.0f + expf(-a)) * b : 0.f);
            }
            bf16* dst = reinterpret_cast<bf16*>(A.out_frag + frag_x_chunk(m, i0 >> 3, MG)) + (i0 & 7);
            *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(ob);
        } else if (EPI == GF_ROPE) {
            const int half = A.d >> 1;
            const int pair0 = (unit * (NT / 2) + set) * 16 + 4 * qq;   // the item's four rotation pairs
            if (m >= A.M || pair0 >= (A.nh + 2 * A.nkv) * half) continue;
            const int hs = pair0 / half, i0 = pair0 % half;   // head slot, dim within its first half (a run of 4 stays inside a head)
            const f32x4 va = reduce4(2 * set, g, l), vb = reduce4(2 * set + 1, g, l);
            float xa[4], xb[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                xa[e] = va[e];
                xb[e] = vb[e];
                if (A.bias != nullptr) {
                    xa[e] += to_f32(A.bias[hs * A.d + i0 + e]);
                    xb[e] += to_f32(A.bias[hs * A.d + i0 + e + half]);
                }
                xa[e] = gf_round(xa[e]);   // the unfused path stores the projection in bfloat16 before it rotates
                xb[e] = gf_round(xb[e]);
            }
            const int slot = A.slots != nullptr ? A.slots[m] : -1;
            if (hs < A.nh + A.nkv) {
                const int p_m = A.pos[m];
                const f32x4 cs = *reinterpret_cast<const f32x4*>(A.cosT + (size_t)p_m * half + i0);
                const f32x4 sn = *reinterpret_cast<const f32x4*>(A.sinT + (size_t)p_m * half + i0);
                bf16 ra[4], rb[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ra[e] = from_f32<bf16>(xa[e] * cs[e] - xb[e] * sn[e]);
                    rb[e] = from_f32<bf16>(xb[e] * cs[e] + xa[e] * sn[e]);
                }
                bf16* dst = nullptr;
                if (hs < A.nh) dst = A.Q + (size_t)m * A.ldq + (size_t)hs * A.d + i0;
                else if (slot >= 0) dst = A.kc + (((size_t)(slot / A.page) * A.nkv + (hs - A.nh)) * A.page + (slot % A.page)) * A.d + i0;
                if (dst != nullptr) {
                    *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(ra);
                    *reinterpret_cast<uint2*>(dst + half) = *reinterpret_cast<const uint2*>(rb);
                }
            } else if (slot >= 0) {
                // values are cached transposed, [pages, nkv, d, page]
                bf16* dst = A.vc + ((size_t)(slot / A.page) * A.nkv + (hs - A.nh - A.nkv)) * A.d * A.page + (slot % A.page);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    dst[(size_t)(i0 + e) * A.page] = from_f32<bf16>(xa[e]);
                    dst[(size_t)(i0 + e + half) * A.page] = from_f32<bf16>(xb[e]);
                }
            }
        } else {   // GF_TAIL
            const int tile = unit * NT + set, n = tile * 16 + 4 * qq;
            float sq = 0.f;
            if (m < A.M && n < A.N) {
                const f32x4 v = reduce4(set, g, l);
                float* rp = A.R + (size_t)m * A.ldr + n;
                bf16 ob[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ob[e] = from_f32<bf16>(0.f);
                    if (n + e < A.N) {
                        const float b_n = A.bias != nullptr ? to_f32(A.bias[n + e]) : 0.f;
                        const float w_n = A.norm_w_f32 ? reinterpret_cast<const float*>(A.norm_w)[n + e]
                                                       : to_f32(reinterpret_cast<const bf16*>(A.norm_w)[n + e]);
                        const float rn = fmaf(A.alpha, v[e] + b_n, rp[e]);
                        rp[e] = rn;
                        ob[e] = from_f32<bf16>(rn * w_n);
                        sq += rn * rn;
                    }
                }
                bf16* dst = reinterpret_cast<bf16*>(A.out_frag + frag_x_chunk(m, n >> 3, MG)) + (n & 7);
                *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(ob);
            }
            // over the four quarters of the tile's rows: neighbouring lanes
            sq += __shfl_xor(sq, 1, 64);
            sq += __shfl_xor(sq, 2, 64);
            if (qq == 0 && m < A.M && tile * 16 < A.N) A.ss_out[(size_t)tile * GF_SS_ROWS + m] = sq;
        }
    }
}

extern "C" int ilm_gemm_frag_ss_rows() { return GF_SS_ROWS; }

static int gf_check(const char* what, const GfArgs& a, int K) {
    ILM_REQUIRE(a.M > 0 && a.M <= 64 && a.N > 0 && K > 0, "%s: needs 1 <= M <= 64, got M=%d N=%d K=%d", what, a.M, a.N, K);
    ILM_REQUIRE(a.Wf != nullptr && a.Xf != nullptr && ((uintptr_t)a.Wf & 15) == 0 && ((uintptr_t)a.Xf & 15) == 0,
                "%s: operands must be 16-byte aligned", what);
    return 0;
}

template <int EPI>
static int gf_launch(const GfArgs& a, int nt, int parts, hipStream_t stream) {
    const int mg = (a.M + 15) / 16;
    const dim3 grid(a.units, parts);
#define GF_GO(MG_, NT_, RD_) gemm_frag_kernel<MG_, NT_, RD_, EPI><<<grid, GF_WAVES * 64, 0, stream>>>(a)
#define GF_MG(NT_, RD_)                       \
    switch (mg) {                             \
        case 1: GF_GO(1, NT_, RD_); break;    \
        case 2: GF_GO(2, NT_, RD_); break;    \
        case 3: GF_GO(3, NT_, RD_); break;    \
        default: GF_GO(4, NT_, RD_); break;   \
    }
    if (nt == 4) { GF_MG(4, 8) } else { GF_MG(2, 16) }
#undef GF_MG
#undef GF_GO
    return 0;
}

// Plain product.  Wf: tiles of W's rows in their own order.  out_kind 0: bfloat16 rows C [M][ldc]; 1: float rows
// or, with steps_per_part < ceil(K / 32), float parts C [parts][M][ldc] part_stride floats apart (bias in part
// 0); 2: bfloat16 in fragment order (out_frag, width N).  nt: tiles a workgroup (2 or 4).
extern "C" int ilm_gemm_frag(void* C, int ldc, long part_stride, int out_kind, const void* Xf, const void* Wf, const void* bias,
                             int M, int N, int K, int steps_per_part, float alpha, int nt, hipStream_t stream) {
    GfArgs a = {};
    a.Wf = (const uint4*)Wf; a.Xf = (const uint4*)Xf; a.bias = (const bf16*)bias;
    a.M = M; a.N = N; a.ksteps = (K + 31) / 32; a.alpha = alpha;
    a.C = C; a.ldc = ldc; a.out_kind = out_kind; a.part_stride = part_stride; a.out_frag = (uint4*)C;
    if (gf_check("gemm_frag", a, K)) return -1;
    ILM_REQUIRE(nt == 2 || nt == 4, "gemm_frag: %d tiles a workgroup", nt);
    ILM_REQUIRE(out_kind >= 0 && out_kind <= 2 && (out_kind == GF_OUT_FRAG || ldc >= N), "gemm_frag: out_kind=%d ldc=%d", out_kind, ldc);
    a.steps_per_part = steps_per_part > 0 && steps_per_part < a.ksteps ? steps_per_part : a.ksteps;
    const int parts = (a.ksteps + a.steps_per_part - 1) / a.steps_per_part;
    ILM_REQUIRE(parts == 1 || out_kind == GF_OUT_F32, "gemm_frag: parts of a split K are float");
    ILM_REQUIRE(parts <= 65535, "gemm_frag: %d parts", parts);
    a.units = ((N + 15) / 16 + nt - 1) / nt;
    gf_launch<GF_PLAIN>(a, nt, parts, stream);
    ILM_LAUNCH_CHECK("gemm_frag");
    return 0;
}

// Gate/up projection with the SwiGLU in its epilogue.  Wf: tiles in pairs (gate rows 16 p .., up rows 16 p ..) of
// W = [Wg; Wu] with I outputs each; bias [2 I] or null.  act_frag: bfloat16 [M][I] in fragment order.  ss: null, or
// the partial sums of squares [ss_tiles][64] of a tail epilogue whose xw is X: rows are divided by
// sqrt(sum / norm_width + eps) first.
extern "C" int ilm_gemm_frag_swiglu(void* act_frag, const void* Xf, const void* Wf, const void* bias, int M, int I, int K,
                                    const void* ss, int ss_tiles, int norm_width, float eps, int nt, hipStream_t stream) {
    GfArgs a = {};
    a.Wf = (const uint4*)Wf; a.Xf = (const uint4*)Xf; a.bias = (const bf16*)bias;
    a.M = M; a.N = I; a.ksteps = (K + 31) / 32; a.steps_per_part = a.ksteps; a.alpha = 1.f;
    a.out_frag = (uint4*)act_frag; a.ss_in = (const float*)ss; a.ss_tiles = ss_tiles; a.norm_width = norm_width; a.eps = eps;
    if (gf_check("gemm_frag_swiglu", a, K)) return -1;
    ILM_REQUIRE(nt == 2 || nt == 4, "gemm_frag_swiglu: %d tiles a workgroup", nt);
    ILM_REQUIRE(ss == nullptr || (ss_tiles > 0 && norm_width > 0 && ((uintptr_t)ss & 15) == 0), "gemm_frag_swiglu: bad sums of squares");
    a.units = ((I + 15) / 16 + nt / 2 - 1) / (nt / 2);
    gf_launch<GF_SWIGLU>(a, nt, 1, stream);
    ILM_LAUNCH_CHECK("gemm_frag_swiglu");
    return 0;
}

// Fused q/k/v projection with rotation and cache write.  Wf: tiles in pairs (first rows, second rows of 16 rotation
// pairs; pair p = head slot p / (d/2), dim p % (d/2); head slots are the q heads, the k heads, the v heads).
// Q [M][ldq] bfloat16 receives the rotated queries; slots null: nothing is cached.
extern "C" int ilm_gemm_frag_rope(void* Q, int ldq, const void* Xf, const void* Wf, const void* bias, int M, int K,
                                  const void* pos, const void* cosT, const void* sinT, void* kc, void* vc, const void* slots,
                                  int nh, int nkv, int d, int page, hipStream_t stream) {
    GfArgs a = {};
    a.Wf = (const uint4*)Wf; a.Xf = (const uint4*)Xf; a.bias = (const bf16*)bias;
    a.M = M; a.N = (nh + 2 * nkv) * d; a.ksteps = (K + 31) / 32; a.steps_per_part = a.ksteps; a.alpha = 1.f;
    a.Q = (bf16*)Q; a.ldq = ldq; a.pos = (const int*)pos; a.cosT = (const float*)cosT; a.sinT = (const float*)sinT;
    a.kc = (bf16*)kc; a.vc = (bf16*)vc; a.slots = (const int*)slots; a.nh = nh; a.nkv = nkv; a.d = d; a.page = page;
    if (gf_check("gemm_frag_rope", a, K)) return -1;
    ILM_REQUIRE(nh > 0 && nkv >= 0 && d > 0 && d % 32 == 0, "gemm_frag_rope: head size %d is not a multiple of 32", d);
    ILM_REQUIRE(ldq >= nh * d && ldq % 4 == 0 && ((uintptr_t)Q & 7) == 0, "gemm_frag_rope: ldq=%d", ldq);
    ILM_REQUIRE(slots == nullptr || (page > 0 && kc != nullptr && vc != nullptr), "gemm_frag_rope: cache missing");
    a.units = ((nh + 2 * nkv) * (d / 2) + 15) / 16;
    gf_launch<GF_ROPE>(a, 2, 1, stream);
    ILM_LAUNCH_CHECK("gemm_frag_rope");
    return 0;
}

// The projection that ends a branch: R [M][ldr] float += alpha (X W^T + bias) in place; xw_frag = bfloat16(R * norm_w)
// in fragment order (width N); ss [ceil(N / 16)][64] partial sums of squares of R's rows (rows beyond M not written).
extern "C" int ilm_gemm_frag_tail(void* R, int ldr, void* xw_frag, void* ss, const void* Xf, const void* Wf, const void* bias,
                                  const void* norm_w, int norm_w_f32, float alpha, int M, int N, int K, int nt,
                                  hipStream_t stream) {
    GfArgs a = {};
    a.Wf = (const uint4*)Wf; a.Xf = (const uint4*)Xf; a.bias = (const bf16*)bias;
    a.M = M; a.N = N; a.ksteps = (K + 31) / 32; a.steps_per_part = a.ksteps; a.alpha = alpha;
    a.R = (float*)R; a.ldr = ldr; a.out_frag = (uint4*)xw_frag; a.ss_out = (float*)ss; a.norm_w = norm_w; a.norm_w_f32 = norm_w_f32;
    if (gf_check("gemm_frag_tail", a, K)) return -1;
    ILM_REQUIRE(nt == 2 || nt == 4, "gemm_frag_tail: %d tiles a workgroup", nt);
    ILM_REQUIRE(R != nullptr && xw_frag != nullptr && ss != nullptr && norm_w != nullptr && ldr >= N, "gemm_frag_tail: null operand or ldr=%d", ldr);
    a.units = ((N + 15) / 16 + nt - 1) / nt;
    gf_launch<GF_TAIL>(a, nt, 1, stream);
    ILM_LAUNCH_CHECK("gemm_frag_tail");
    return 0;
}
