// Entry points that allocate nothing.
//
// They have no counterpart in the reference.  They are for callers that cannot call hipMalloc: code
// under HIP graph capture, tight serving loops, harnesses that forbid allocation.  Such a caller
// passes inputs and outputs only; what the kernels need beyond them lies in a file-scope device
// array of fixed size that every GPU the library runs on holds until the process ends.
#pragma once
#include <hip/hip_runtime.h>

// Floats of the static scratch of ilm_attn_mfma_static: 4 Mi floats = 16 MiB a GPU.
#define ILM_ATTN_SCRATCH_FLOATS (4l << 20)

extern "C" {

// ilm_attn_mfma (chunked single-token paged attention, bfloat16) without its two workspace
// arguments: the chunks' partial results (unnormalised outputs, maxima and sums) go to the static
// scratch.  Needs T * nh * nsplit * (d + 2) <= ILM_ATTN_SCRATCH_FLOATS floats (64 tokens x 32 heads x
// 16 chunks x 130 at most, for instance); beyond that it returns -1 with a message and launches
// nothing.  With nsplit == 1 the scratch is not used.  It calls no hipMalloc, hipFree or other
// allocating routine; the scratch's address is looked up once per device: by ilm_attn_static_init(), or
// else at the first call with that device current (a caller that records HIP graphs calls
// ilm_attn_static_init() before its first capture on a device, so that the look-up, which is no stream
// operation, does not fall into a capture).  Every slot the merge kernel reads is written by the attention kernel of the
// same call, so nothing has to be cleared between calls.  All calls on one GPU share that GPU's
// scratch: calls that overlap on one GPU (two streams, two threads) race; calls on one stream are
// ordered and safe.  Arguments, results and return value otherwise as ilm_attn_mfma.
int ilm_attn_mfma_static(void* out, const void* q, const void* kc, const void* vc, const void* block_tables,
                         const void* seg, const void* pos, const void* rows, int T, int nh, int nkv, int d,
                         int page, int max_blocks, int q_stride, int out_stride, float scale, int window,
                         int nsplit, int span, hipStream_t stream);

// Looks up the scratch's address on the current device (once; later calls return at once).  0, or -1
// with a message.  Allocates nothing.
int ilm_attn_static_init();

// ILM_ATTN_SCRATCH_FLOATS, for callers that size their calls at run time.
long ilm_attn_static_scratch_floats();

}
