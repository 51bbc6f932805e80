// Sampling from rows of float logits: argmax, and temperature / top-k / top-p with an inverse CDF.
//
// Definition: temperature == 0 or top_k == 1 -> the first index of the maximum.  Otherwise
// e_i = exp((l_i - max) / temperature); keep the top_k largest logits (0 or >= V keeps all; ties
// with the k-th value are kept); among those keep the fewest largest whose mass reaches top_p of
// the kept mass (ties kept); the token is the first index, in vocabulary order over the kept set,
// whose running mass exceeds u * (kept mass), u in [0, 1) supplied by the host per row.
// Thresholds are found by building the k-th largest value bit by bit over an order-preserving
// integer image of the floats, so no sort and no scratch memory is needed; one block per row.
#include "common.h"

#define SB 1024
#define SNW (SB / 64)

__device__ __forceinline__ uint32_t okey(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ void better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) {
        bv = v;
        bi = i;
    }
}

// argmax of one row by the whole block (first index on ties); result valid in every thread
__device__ int block_argmax(const float* __restrict__ row, int V, float* sv, int* si, float* out_max) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    if ((V & 3) == 0 && ((uintptr_t)row & 15) == 0) {
        // 16-byte loads, four of them in flight a thread: the scan is bound by memory latency
        const float4* row4 = reinterpret_cast<const float4*>(row);
        const int V4 = V >> 2;
        for (int i = threadIdx.x; i < V4; i += 4 * SB) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = i + u * SB;
                v[u] = row4[j < V4 ? j : V4 - 1];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = i + u * SB;
                if (j < V4) {
                    better(bv, bi, v[u].x, 4 * j);
                    better(bv, bi, v[u].y, 4 * j + 1);
                    better(bv, bi, v[u].z, 4 * j + 2);
                    better(bv, bi, v[u].w, 4 * j + 3);
                }
            }
        }
    } else {
        for (int i = threadIdx.x; i < V; i += SB) better(bv, bi, row[i], i);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(bv, o, 64);
        int oi = __shfl_xor(bi, o, 64);
        better(bv, bi, ov, oi);
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) {
        sv[w] = bv;
        si[w] = bi;
    }
    __syncthreads();
    bv = sv[0];
    bi = si[0];
    for (int i = 1; i < SNW; ++i) better(bv, bi, sv[i], si[i]);
    if (bi == 0x7fffffff) bi = 0;  // a row of NaN
    *out_max = bv;
    return bi;
}

__global__ void __launch_bounds__(SB)
argmax_kernel(int* __restrict__ out, const float* __restrict__ logits, int V, int stride) {
    __shared__ float sv[SNW];
    __shared__ int si[SNW];
    float mx;
    const int bi = block_argmax(logits + (size_t)blockIdx.x * stride, V, sv, si, &mx);
    if (threadIdx.x == 0) out[blockIdx.x] = bi;
}

extern "C" int ilm_argmax(void* out, const void* logits, int n, int V, int stride,
                          hipStream_t stream) {
    ILM_REQUIRE(n > 0 && V > 0 && stride >= V, "argmax: bad sizes n=%d V=%d stride=%d", n, V, stride);
    argmax_kernel<<<n, SB, 0, stream>>>((int*)out, (const float*)logits, V, stride);
    ILM_LAUNCH_CHECK("argmax");
    return 0;
}

__device__ __forceinline__ float block_sum_f(float v, float* red) { return block_sum<SNW>(v, red); }

__device__ __forceinline__ int block_sum_i(int v, int* red) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int i = 0; i < SNW; ++i) t += red[i];
    return t;
}

__global__ void __launch_bounds__(SB)
sample_kernel(int* __restrict__ out, const float* __restrict__ logits, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const float* __restrict__ uniform, int V, int stride) {
    __shared__ float sv[SNW];
    __shared__ int si[SNW];
    __shared__ float redf[SNW];
    __shared__ int redi[SNW];
    __shared__ float wave_tot[SNW];
    __shared__ int claim;
    __shared__ int last_kept;
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * stride;
    const float temp = temperature[r];
    const int k = top_k[r];
    const float pp = top_p[r];
    float mx;
    const int amax = block_argmax(row, V, sv, si, &mx);
    if (temp == 0.0f || k == 1) {
        if (threadIdx.x == 0) out[r] = amax;
        return;
    }
    const float inv_t = 1.0f / temp;

    // threshold of the top-k: the k-th largest key
    uint32_t tau = 0u;
    if (k > 0 && k < V) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tau | (1u << bit);
            int c = 0;
            for (int i = threadIdx.x; i < V; i += SB) c += okey(row[i]) >= cand;
            if (block_sum_i(c, redi) >= k) tau = cand;
        }
    }
    // threshold of the top-p within the kept set
    if (pp < 1.0f) {
        float sk = 0.f;
        for (int i = threadIdx.x; i < V; i += SB)
            if (okey(row[i]) >= tau) sk += expf((row[i] - mx) * inv_t);
        sk = block_sum_f(sk, redf);
        const float need = pp * sk;
        uint32_t tp = 0u;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tp | (1u << bit);
            const uint32_t thr = cand > tau ? cand : tau;
            float ms = 0.f;
            for (int i = threadIdx.x; i < V; i += SB)
                if (okey(row[i]) >= thr) ms += expf((row[i] - mx) * inv_t);
            if (block_sum_f(ms, redf) >= need) tp = cand;
        }
        if (tp > tau) tau = tp;
    }
    // inverse CDF in vocabulary order over the kept set
    const int chunk = (V + SB - 1) / SB;
    const int i0 = threadIdx.x * chunk;
    const int i1 = (i0 + chunk < V) ? i0 + chunk : V;
    float local = 0.f;
    int my_last = -1;
    for (int i = i0; i < i1; ++i)
        if (okey(row[i]) >= tau) {
            local += expf((row[i] - mx) * inv_t);
            my_last = i;
        }
    // inclusive scan of `local` over the block
    float incl = local;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float n = __shfl_up(incl, o, 64);
        if (lane >= o) incl += n;
    }
    if (threadIdx.x == 0) {
        claim = 0x7fffffff;
        last_kept = -1;
    }
    __syncthreads();
    if (lane == 63) wave_tot[w] = incl;
    __syncthreads();
    float before = 0.f, total = 0.f;
    for (int i = 0; i < SNW; ++i) {
        if (i < w) before += wave_tot[i];
        total += wave_tot[i];
    }
    incl += before;
    const float target = uniform[r] * total;
    if (local > 0.f && target < incl) atomicMin(&claim, (int)threadIdx.x);
    if (my_last >= 0) atomicMax(&last_kept, my_last);
    __syncthreads();
    if (claim == 0x7fffffff) {
        if (threadIdx.x == 0) out[r] = last_kept >= 0 ? last_kept : amax;
        return;
    }
    if ((int)threadIdx.x == claim) {
        float cum = incl - local;
        int pick = my_last;
        for (int i = i0; i < i1; ++i)
            if (okey(row[i]) >= tau) {
                cum += expf((row[i] - mx) * inv_t);
                if (target < cum) {
                    pick = i;
                    break;
                }
            }
        out[r] = pick;
    }
}

// The same definition with the row held in registers: every thread keeps the order-preserving keys
// of elements tid, tid + SB, ... (EPT of them), so the 32 + 32 rounds of the two threshold searches
// read nothing from memory.  The exponentials of the top-p search are recomputed from the keys, and
// skipped where no lane of a wave holds a kept element (with a small top-k nearly everywhere).
__device__ __forceinline__ float key_to_float(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

template <int NW>
__device__ __forceinline__ int block_sum_i_n(int v, int* red) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int i = 0; i < NW; ++i) t += red[i];
    return t;
}

template <int NW>
__device__ __forceinline__ uint32_t block_max_u(uint32_t v, uint32_t* red) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t x = __shfl_xor(v, o, 64);
        v = x > v ? x : v;
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    uint32_t t = 0;
#pragma unroll
    for (int i = 0; i < NW; ++i) t = red[i] > t ? red[i] : t;
    return t;
}

template <int EPT, int NTH>
__global__ void __launch_bounds__(NTH)
sample_reg_kernel(int* __restrict__ out, const float* __restrict__ logits, const float* __restrict__ temperature,
                  const int* __restrict__ top_k, const float* __restrict__ top_p,
                  const float* __restrict__ uniform, int V, int stride) {
    constexpr int NW = NTH / 64;
    __shared__ float redf[NW];
    __shared__ int redi[NW];
    __shared__ uint32_t redu[NW];
    __shared__ int last_kept;
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * stride;
    const float temp = temperature[r];
    const int k = top_k[r];
    const float pp = top_p[r];
    uint32_t keys[EPT];   // 0 (below every number) beyond the row
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int i = threadIdx.x + e * NTH;
        const float v = row[i < V ? i : V - 1];
        keys[e] = i < V ? okey(v) : 0u;
    }
    uint32_t kmax = 0u;
#pragma unroll
    for (int e = 0; e < EPT; ++e) kmax = keys[e] > kmax ? keys[e] : kmax;
    kmax = block_max_u<NW>(kmax, redu);
    // the first index that holds the maximum
    int first = 0x7fffffff;
#pragma unroll
    for (int e = EPT - 1; e >= 0; --e)
        if (keys[e] == kmax) first = threadIdx.x + e * NTH;
    // min over the block as a max of the complement (index 0 becomes the largest value)
    first = 0x7fffffff - (int)block_max_u<NW>((uint32_t)(0x7fffffff - first), redu);
    if (first == 0x7fffffff) first = 0;
    if (temp == 0.0f || k == 1) {
        if (threadIdx.x == 0) out[r] = first;
        return;
    }
    const float mx = key_to_float(kmax);
    const float inv_t = 1.0f / temp;
    uint32_t tau = 0u;
    if (k > 0 && k < V) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tau | (1u << bit);
            int c = 0;
#pragma unroll
            for (int e = 0; e < EPT; ++e) c += keys[e] >= cand;
            if (block_sum_i_n<NW>(c, redi) >= k) tau = cand;
        }
    }
    if (tau == 0u) tau = 1u;   // keys of real elements are above 0; the padding is not kept
    if (pp < 1.0f) {
        // mass of the elements with key >= thr (hardware exp2: the search needs the order of masses,
        // the draw below uses expf)
        const float inv_t2 = inv_t * 1.4426950408889634f;
        auto mass = [&](uint32_t thr) -> float {
            float ms = 0.f;
            constexpr int GRP = 8;   // one branch for eight elements: kept ones are rare under a top-k
#pragma unroll
            for (int e0 = 0; e0 < EPT; e0 += GRP) {
                uint32_t ke[GRP];
                bool any = false;
#pragma unroll
                for (int g = 0; g < GRP; ++g) {
                    ke[g] = e0 + g < EPT ? keys[e0 + g] : 0u;
                    asm volatile("" : "+v"(ke[g]));   // the exponentials stay inside the rounds: outside they would need EPT more registers
                    any = any || ke[g] >= thr;
                }
                if (__builtin_amdgcn_ballot_w64(any) != 0ull) {
#pragma unroll
                    for (int g = 0; g < GRP; ++g)
                        ms += ke[g] >= thr ? __builtin_amdgcn_exp2f((key_to_float(ke[g]) - mx) * inv_t2) : 0.f;
                }
            }
            return block_sum<NW>(ms, redf);
        };
        const float need = pp * mass(tau);
        uint32_t tp = 0u;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tp | (1u << bit);
            if (mass(cand > tau ? cand : tau) >= need) tp = cand;
        }
        if (tp > tau) tau = tp;
    }
    // Inverse CDF in vocabulary order over the kept set, from the registers: element e of thread
    // (w, lane) has index e * NTH + w * 64 + lane, so vocabulary order is (e, w, lane).  Every wave
    // leaves the kept mass of each of its 64-element runs in LDS; wave 0 finds the run that holds
    // u * total; the wave that owns it finds the lane.
    __shared__ float run_mass[EPT][NW];
    __shared__ int pick_e, pick_w;
    __shared__ float pick_before, pick_target;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int my_last = -1;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const bool in = keys[e] >= tau;
        float m = 0.f;
        if (__builtin_amdgcn_ballot_w64(in) != 0ull) {
            m = in ? expf((key_to_float(keys[e]) - mx) * inv_t) : 0.f;
            m = wave_sum(m);
        }
        if (lane == 0) run_mass[e][w] = m;
        if (in) my_last = threadIdx.x + e * NTH;
    }
    if (threadIdx.x == 0) {
        last_kept = -1;
        pick_e = -1;
    }
    __syncthreads();
    if (my_last >= 0) atomicMax(&last_kept, my_last);
    if (w == 0) {
        // runs in order, a contiguous stretch of them per lane
        constexpr int NRUN = EPT * NW;
        constexpr int PER = (NRUN + 63) / 64;
        const float* rm = &run_mass[0][0];
        float mine = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int j = lane * PER + i;
            mine += j < NRUN ? rm[j] : 0.f;
        }
        float incl = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float n = __shfl_up(incl, o, 64);
            if (lane >= o) incl += n;
        }
        const float total = __shfl(incl, 63, 64);
        const float target = uniform[r] * total;
        const bool here = mine > 0.f && target < incl;
        const unsigned long long bal = __builtin_amdgcn_ballot_w64(here);
        if (bal != 0ull && lane == __builtin_ctzll(bal)) {
            float cum = incl - mine;
            for (int i = 0; i < PER; ++i) {
                const int j = lane * PER + i;
                if (j >= NRUN) break;
                if (rm[j] > 0.f && target < cum + rm[j]) {
                    pick_e = j / NW;
                    pick_w = j % NW;
                    pick_before = cum;
                    pick_target = target;
                    break;
                }
                cum += rm[j];
            }
        }
    }
    __syncthreads();
    if (pick_e < 0) {   // rounding left u * total at or beyond the sum: the last kept element
        if (threadIdx.x == 0) out[r] = last_kept >= 0 ? last_kept : first;
        return;
    }
    if (w == pick_w) {
        float m = 0.f;
        const int pe = pick_e;
        uint32_t ke = 0u;
#pragma unroll
        for (int e = 0; e < EPT; ++e) ke = e == pe ? keys[e] : ke;
        const bool in = ke >= tau;
        m = in ? expf((key_to_float(ke) - mx) * inv_t) : 0.f;
        float incl = m;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float n = __shfl_up(incl, o, 64);
            if (lane >= o) incl += n;
        }
        const bool here = in && pick_target < pick_before + incl;
        const unsigned long long bal = __builtin_amdgcn_ballot_w64(here);
        // the run holds the target by the sum of its masses; a different order of summation may
        // leave it just short: then the run's last kept element
        const unsigned long long kept = __builtin_amdgcn_ballot_w64(in);
        const int pl = bal != 0ull ? __builtin_ctzll(bal) : 63 - __builtin_clzll(kept);
        if (lane == 0) out[r] = pe * NTH + w * 64 + pl;
    }
}

extern "C" int ilm_sample(void* out, const void* logits, const void* temperature, const void* top_k,
                          const void* top_p, const void* uniform, int n, int V, int stride,
                          hipStream_t stream) {
    ILM_REQUIRE(n > 0 && V > 0 && stride >= V, "sample: bad sizes n=%d V=%d stride=%d", n, V, stride);
#define SAMPLE_ARGS (int*)out, (const float*)logits, (const float*)temperature, (const int*)top_k, (const float*)top_p, \
                    (const float*)uniform, V, stride
    // rows of up to 192 * 512 numbers are held in registers; longer ones are read again every round
    if (V <= 16 * 1024) sample_reg_kernel<16, 1024><<<n, 1024, 0, stream>>>(SAMPLE_ARGS);
    else if (V <= 32 * 1024) sample_reg_kernel<32, 1024><<<n, 1024, 0, stream>>>(SAMPLE_ARGS);
    else if (V <= 96 * 512) sample_reg_kernel<96, 512><<<n, 512, 0, stream>>>(SAMPLE_ARGS);
    else if (V <= 144 * 512) sample_reg_kernel<144, 512><<<n, 512, 0, stream>>>(SAMPLE_ARGS);
    else if (V <= 192 * 512) sample_reg_kernel<192, 512><<<n, 512, 0, stream>>>(SAMPLE_ARGS);
    else sample_kernel<<<n, SB, 0, stream>>>(SAMPLE_ARGS);
#undef SAMPLE_ARGS
    ILM_LAUNCH_CHECK("sample");
    return 0;
}
