// Paged attention on the matrix cores (bfloat16 in, float softmax and accumulation).
//
// Same contract as attn_basic.hip.  One wave serves one token and one group of up to 16 query
// heads that share a KV head, over one chunk of ATT_CHUNK keys; chunks are aligned to absolute key
// index, so what is summed in which order depends on (request, position) alone.  With more than
// one chunk the partial results (max, sum, unnormalised output) go to a workspace and a second
// kernel merges them in chunk order.
//
// Per 32 keys:  S^T[keys x heads] = K Q^T   (v_mfma_f32_16x16x32_bf16, K rows on the A side, read
//                                            straight from the cache; d is the reduced dimension)
//               online softmax in float, per head = per lane column
//               O^T[d x heads] += V^T P^T   (V is cached transposed, [d][page], so that 8
//                                            consecutive keys of one dim are one 16-byte load)
// The rows of the two S tiles are assigned to keys so that each lane ends up with the
// probabilities of 8 consecutive keys: they feed the second product without leaving registers.
// Needs: head size a multiple of 16 up to 128, page size a multiple of 16.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define ATT_CHUNK 256
#define NEG_BIG (-1.0e30f)

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}

template <int D16>
__global__ void __launch_bounds__(64)
attn_mfma_kernel(bf16* __restrict__ out, float* __restrict__ ws_acc, float* __restrict__ ws_ml,
                 const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                 const int* __restrict__ block_tables, const int* __restrict__ seg,
                 const int* __restrict__ pos, int nh, int nkv, int page, int max_blocks, int q_stride,
                 int out_stride, float scale_log2e, int window, int nsplit) {
    constexpr int D = D16 * 16;
    constexpr int KS = (D + 31) / 32;
    const int t = blockIdx.x;
    const int G = nh / nkv;
    const int HG = (G + 15) / 16;
    const int kvh = blockIdx.y / HG, hg = blockIdx.y % HG;
    const int split = blockIdx.z;
    const int lane = threadIdx.x, r = lane & 15, qg = lane >> 4;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int hcol = hg * 16 + r;
    const bool head_ok = hcol < G;
    const int head = kvh * G + (head_ok ? hcol : G - 1);

    int k_begin = split * ATT_CHUNK;
    int k_end = k_begin + ATT_CHUNK;
    if (k_begin < lo) k_begin = lo;
    if (k_end > p + 1) k_end = p + 1;
    if (k_begin >= k_end) {
        if (nsplit > 1 && head_ok && qg == 0) {
            float* ml = ws_ml + (((size_t)t * nh + head) * nsplit + split) * 2;
            ml[0] = NEG_BIG;
            ml[1] = 0.f;
        }
        return;
    }
    const int* bt = block_tables + (size_t)seg[t] * max_blocks;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    uint4 qf[KS];
    const bf16* qrow = q + (size_t)t * q_stride + (size_t)head * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int dofs = ks * 32 + qg * 8;
        qf[ks] = (dofs < D) ? *reinterpret_cast<const uint4*>(qrow + dofs) : zero4;
    }
    f32x4 acc[D16];
#pragma unroll
    for (int db = 0; db < D16; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = NEG_BIG, lsum = 0.f;

    for (int kb = k_begin & ~31; kb < k_end; kb += 32) {
        // ---- S^T = K Q^T for two tiles of 16 keys; row i of tile tau is key kb + (i/4)*8 + tau*4 + i%4
        f32x4 s[2];
#pragma unroll
        for (int tau = 0; tau < 2; ++tau) {
            int key = kb + (r >> 2) * 8 + tau * 4 + (r & 3);
            key = key < k_begin ? k_begin : (key >= k_end ? k_end - 1 : key);  // stay on pages that exist
            const int pg = bt[key / page];
            const bf16* krow = kc + (((size_t)pg * nkv + kvh) * page + (key % page)) * D;
            s[tau] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int dofs = ks * 32 + qg * 8;
                const uint4 kf = (dofs < D) ? *reinterpret_cast<const uint4*>(krow + dofs) : zero4;
                s[tau] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf),
                                                                 __builtin_bit_cast(bf16x8, qf[ks]), s[tau], 0, 0, 0);
            }
        }
        // lane (r, qg) now holds, for head column r, keys kb + qg*8 + tau*4 + e
        float sv[8];
        float mx = NEG_BIG;
#pragma unroll
        for (int tau = 0; tau < 2; ++tau)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = kb + qg * 8 + tau * 4 + e;
                const bool ok = key >= k_begin && key < k_end;
                const float v = ok ? s[tau][e] * scale_log2e : NEG_BIG;
                sv[tau * 4 + e] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);
        const float corr = __builtin_amdgcn_exp2f(m - m_new);
        float pe[8];
        float rs = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            pe[j] = (sv[j] > 0.5f * NEG_BIG) ? __builtin_amdgcn_exp2f(sv[j] - m_new) : 0.f;
            rs += pe[j];
        }
        rs += __shfl_xor(rs, 16, 64);
        rs += __shfl_xor(rs, 32, 64);
        lsum = lsum * corr + rs;
        m = m_new;
        uint4 pf;
        pf.x = pack_bf16x2(pe[0], pe[1]);
        pf.y = pack_bf16x2(pe[2], pe[3]);
        pf.z = pack_bf16x2(pe[4], pe[5]);
        pf.w = pack_bf16x2(pe[6], pe[7]);
        // ---- O^T += V^T P^T; this lane's 8 keys are kb + qg*8 .. +8, on one page
        const int key0 = kb + qg * 8;
        const bool vok = key0 < k_end && key0 + 8 > k_begin;
        const bf16* vbase = nullptr;
        if (vok) {
            const int pg = bt[key0 / page];
            vbase = vc + ((size_t)pg * nkv + kvh) * D * page + (key0 % page);
        }
#pragma unroll
        for (int db = 0; db < D16; ++db) {
            const uint4 vf = vok ? *reinterpret_cast<const uint4*>(vbase + (size_t)(db * 16 + r) * page) : zero4;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[db][e] *= corr;
            acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf),
                                                             __builtin_bit_cast(bf16x8, pf), acc[db], 0, 0, 0);
        }
    }
    // acc[db][e] is dim db*16 + qg*4 + e of head column r
    if (!head_ok) return;
    if (nsplit == 1) {
        const float inv = 1.0f / lsum;
        bf16* orow = out + (size_t)t * out_stride + (size_t)head * D;
#pragma unroll
        for (int db = 0; db < D16; ++db) {
            uint2 w;
            w.x = pack_bf16x2(acc[db][0] * inv, acc[db][1] * inv);
            w.y = pack_bf16x2(acc[db][2] * inv, acc[db][3] * inv);
            *reinterpret_cast<uint2*>(orow + db * 16 + qg * 4) = w;
        }
    } else {
        const size_t slot = ((size_t)t * nh + head) * nsplit + split;
        float* wa = ws_acc + slot * D;
#pragma unroll
        for (int db = 0; db < D16; ++db)
            *reinterpret_cast<f32x4*>(wa + db * 16 + qg * 4) = acc[db];
        if (qg == 0) {
            ws_ml[slot * 2] = m;
            ws_ml[slot * 2 + 1] = lsum;
        }
    }
}

// out[t, h, :] = sum_i acc_i 2^(m_i - M) / sum_i l_i 2^(m_i - M), chunks in ascending order
__global__ void __launch_bounds__(64)
attn_merge_kernel(bf16* __restrict__ out, const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
                  const int* __restrict__ pos, int nh, int D, int out_stride, int window, int nsplit) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int s_lo = lo / ATT_CHUNK, s_hi = p / ATT_CHUNK;
    const size_t base = ((size_t)t * nh + h) * nsplit;
    float M = NEG_BIG;
    for (int s = s_lo; s <= s_hi; ++s) M = fmaxf(M, ws_ml[(base + s) * 2]);
    float L = 0.f;
    for (int s = s_lo; s <= s_hi; ++s) L += ws_ml[(base + s) * 2 + 1] * __builtin_amdgcn_exp2f(ws_ml[(base + s) * 2] - M);
    const float inv = 1.0f / L;
    for (int dd = lane; dd < D; dd += 64) {
        float o = 0.f;
        for (int s = s_lo; s <= s_hi; ++s)
            o += ws_acc[(base + s) * D + dd] * __builtin_amdgcn_exp2f(ws_ml[(base + s) * 2] - M);
        out[(size_t)t * out_stride + (size_t)h * D + dd] = from_f32<bf16>(o * inv);
    }
}

extern "C" int ilm_attn_mfma_chunk() { return ATT_CHUNK; }

extern "C" int ilm_attn_mfma(void* out, void* ws_acc, void* ws_ml, const void* q, const void* kc,
                             const void* vc, const void* block_tables, const void* seg, const void* pos,
                             int T_, int nh, int nkv, int d, int page, int max_blocks, int q_stride,
                             int out_stride, float scale, int window, int nsplit, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn_mfma: bad head counts nh=%d nkv=%d", nh, nkv);
    ILM_REQUIRE(d % 16 == 0 && d >= 16 && d <= 128, "attn_mfma: head size %d is not a multiple of 16 up to 128", d);
    ILM_REQUIRE(page % 16 == 0 && page > 0, "attn_mfma: page size %d is not a multiple of 16", page);
    ILM_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0 && ((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 7) == 0,
                "attn_mfma: q and out rows must be 16-byte / 8-byte aligned");
    ILM_REQUIRE(nsplit >= 1 && (nsplit == 1 || (ws_acc != nullptr && ws_ml != nullptr)), "attn_mfma: workspace missing");
    const int G = nh / nkv, HG = (G + 15) / 16;
    ILM_REQUIRE(nkv * HG <= 65535 && nsplit <= 65535, "attn_mfma: grid too large");
    dim3 grid(T_, nkv * HG, nsplit);
    const float sl2 = scale * 1.4426950408889634f;
#define AM_CASE(D16)                                                                                           \
    case D16:                                                                                                  \
        attn_mfma_kernel<D16><<<grid, 64, 0, stream>>>((bf16*)out, (float*)ws_acc, (float*)ws_ml, (const bf16*)q, \
                                                       (const bf16*)kc, (const bf16*)vc, (const int*)block_tables, \
                                                       (const int*)seg, (const int*)pos, nh, nkv, page, max_blocks, \
                                                       q_stride, out_stride, sl2, window, nsplit);             \
        break
    switch (d / 16) {
        AM_CASE(1); AM_CASE(2); AM_CASE(3); AM_CASE(4); AM_CASE(5); AM_CASE(6); AM_CASE(7); AM_CASE(8);
        default: ILM_REQUIRE(false, "attn_mfma: head size %d", d);
    }
#undef AM_CASE
    ILM_LAUNCH_CHECK("attn_mfma");
    if (nsplit > 1) {
        dim3 g2(T_, nh);
        attn_merge_kernel<<<g2, 64, 0, stream>>>((bf16*)out, (const float*)ws_acc, (const float*)ws_ml, (const int*)pos,
                                                 nh, d, out_stride, window, nsplit);
        ILM_LAUNCH_CHECK("attn_merge");
    }
    return 0;
}
