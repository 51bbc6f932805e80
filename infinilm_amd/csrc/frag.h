// Fragment order: operands of v_mfma_f32_16x16x32_bf16 laid out in memory the way the instruction takes
// them, so that the 64 lanes of a wave load a fragment as 1 KB of consecutive bytes.
//
// A fragment is 16 rows x 32 k of bfloat16: lane (r = lane % 16, q = lane / 16) holds row r, k 8 q .. 8 q + 7,
// 16 bytes.  Loaded straight from row-major memory, such a fragment touches 16 rows and half a 128-byte line
// of each, and a compute unit takes in about 36 GB/s that way (9 TB/s over the chip, measured with reads
// that hit L2); in fragment order the same unit takes in 130 GB/s.  For W read once from memory the first
// is bearable; for X, which every workgroup reads again from the L2s, it is not; and with both in fragment
// order the products of a decode step stream W near the memory's own speed.
//
//   weights      Wf[tile][step][lane]   16 bytes each; tile = 16 rows of W (in an order the consumer's epilogue
//                                       likes: see the packers), step = 32 k; rows and k beyond W are zeros
//   activations  Xf[step][group][lane]  group = 16 rows of X, MG = ceil(M / 16) groups; k beyond K is zeros,
//                                       rows beyond M are never read into a result that is kept
#pragma once
#include <stddef.h>

// index of the 16-byte chunk that holds X[m][8 k8 .. 8 k8 + 7] (MG groups of rows)
__device__ __host__ __forceinline__ size_t frag_x_chunk(int m, int k8, int MG) {
    return ((size_t)(k8 >> 2) * MG + (m >> 4)) * 64 + (size_t)((k8 & 3) * 16 + (m & 15));
}
