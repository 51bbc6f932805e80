// Packers into fragment order (frag.h): weights once after loading, activations where a producer has no
// fragment-order store of its own.
#include "common.h"
#include "frag.h"

// dst[tile][step][lane] <- src row `rows[tile * 16 + lane % 16]` (or tile * 16 + lane % 16 without a row list),
// k 32 step + 8 (lane / 16) ..; rows < 0 or >= N and k >= K give zeros.  A thread a chunk.
__global__ void __launch_bounds__(256)
frag_pack_weight_kernel(uint4* __restrict__ dst, const bf16* __restrict__ src, const int* __restrict__ rows, int N, int K,
                        int ldw, int tiles, int ksteps) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)tiles * ksteps * 64) return;
    const int lane = idx & 63, r = lane & 15, q = lane >> 4;
    const int step = (idx >> 6) % ksteps, tile = (idx >> 6) / ksteps;
    const int out_row = tile * 16 + r;
    const int row = rows != nullptr ? rows[out_row] : out_row;
    const int k = 32 * step + 8 * q;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (row >= 0 && row < N && k < K) v = *reinterpret_cast<const uint4*>(src + (size_t)row * ldw + k);
    dst[idx] = v;
}

// dst[step][group][lane] <- src[16 group + lane % 16][32 step + 8 (lane / 16) ..]; rows >= M and k >= K give zeros
__global__ void __launch_bounds__(256)
frag_pack_rows_kernel(uint4* __restrict__ dst, const bf16* __restrict__ src, int M, int K, int ld, int MG, int ksteps) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)ksteps * MG * 64) return;
    const int lane = idx & 63, r = lane & 15, q = lane >> 4;
    const int g = (idx >> 6) % MG, step = (idx >> 6) / MG;
    const int m = 16 * g + r, k = 32 * step + 8 * q;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (m < M && k < K) v = *reinterpret_cast<const uint4*>(src + (size_t)m * ld + k);
    dst[idx] = v;
}

// the reverse, for tests and for consumers that take plain rows
__global__ void __launch_bounds__(256)
frag_unpack_rows_kernel(bf16* __restrict__ dst, const uint4* __restrict__ src, int M, int K, int ld, int MG) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int k8s = K >> 3;
    if (idx >= (size_t)M * k8s) return;
    const int m = idx / k8s, k8 = idx % k8s;
    *reinterpret_cast<uint4*>(dst + (size_t)m * ld + 8 * k8) = src[frag_x_chunk(m, k8, MG)];
}

extern "C" int ilm_frag_pack_weight(void* dst, const void* src, const void* rows, int N, int K, int ldw, int tiles,
                                    hipStream_t stream) {
    ILM_REQUIRE(N > 0 && K > 0 && tiles > 0 && K % 8 == 0 && ldw % 8 == 0 && ldw >= K, "frag_pack_weight: N=%d K=%d ldw=%d tiles=%d",
                N, K, ldw, tiles);
    ILM_REQUIRE(((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0, "frag_pack_weight: operands must be 16-byte aligned");
    const int ksteps = (K + 31) / 32;
    const size_t chunks = (size_t)tiles * ksteps * 64;
    frag_pack_weight_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, stream>>>((uint4*)dst, (const bf16*)src, (const int*)rows,
                                                                                 N, K, ldw, tiles, ksteps);
    ILM_LAUNCH_CHECK("frag_pack_weight");
    return 0;
}

extern "C" int ilm_frag_pack_rows(void* dst, const void* src, int M, int K, int ld, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && K > 0 && K % 8 == 0 && ld % 8 == 0 && ld >= K, "frag_pack_rows: M=%d K=%d ld=%d", M, K, ld);
    ILM_REQUIRE(((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0, "frag_pack_rows: operands must be 16-byte aligned");
    const int MG = (M + 15) / 16, ksteps = (K + 31) / 32;
    const size_t chunks = (size_t)ksteps * MG * 64;
    frag_pack_rows_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, stream>>>((uint4*)dst, (const bf16*)src, M, K, ld, MG, ksteps);
    ILM_LAUNCH_CHECK("frag_pack_rows");
    return 0;
}

extern "C" int ilm_frag_unpack_rows(void* dst, const void* src, int M, int K, int ld, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && K > 0 && K % 8 == 0 && ld % 8 == 0 && ld >= K, "frag_unpack_rows: M=%d K=%d ld=%d", M, K, ld);
    const size_t chunks = (size_t)M * (K / 8);
    frag_unpack_rows_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, stream>>>((bf16*)dst, (const uint4*)src, M, K, ld, (M + 15) / 16);
    ILM_LAUNCH_CHECK("frag_unpack_rows");
    return 0;
}
