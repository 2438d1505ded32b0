// Decode attention for callers that cannot allocate device memory.
//
// This entry point has no counterpart in the reference (izmttk/ullm takes its attention from a
// library that is handed a workspace tensor).  It is for callers that may not call hipMalloc: code
// under HIP graph capture, tight serving loops, harnesses that forbid allocation.
//
// ullm_attention_decode (attention_mfma.hip) cuts a token's keys over several blocks and needs a
// workspace of ullm_attention_decode_workspace(...) floats for the blocks' partial results, which the
// caller has to allocate.  ullm_attention_decode_static is the same operation with the same kernels,
// but the partial results go to a file-scope device array of ULLM_DECODE_SCRATCH_FLOATS floats
// (ULLM_DECODE_SCRATCH_FLOATS * 4 bytes = 8 MiB, held by every GPU the library runs on until the
// process ends).  The caller still passes inputs and outputs; nothing is allocated or freed, here or
// in a library routine.
//
// * A call whose partial results need more than ULLM_DECODE_SCRATCH_FLOATS floats
//   (n_items * nq * num_splits * (hd + 4)) is refused with ULLM_ERR_SCRATCH; nothing is launched.
// * The array's device address is looked up once per device, with that device current, at the first
//   call on it (hipGetSymbolAddress); a failure of that lookup is returned as its hipError_t.  The lookup
//   is not stream-ordered and may load the code object: it must not happen while a stream is capturing.
//   A caller that captures calls ullm_attention_decode_static_capacity() (or the entry point itself) once
//   on the device beforehand; every later call only launches kernels on the given stream.
// * All calls on one GPU share that GPU's array.  Every float a call reads it has written itself in
//   the same call (the reduce kernel reads exactly the rows the split kernel stored), so nothing
//   needs clearing between calls; but two calls that overlap in time on one GPU (different streams,
//   or two graphs replayed side by side) race on the array and give wrong results.  Serialise them.
#pragma once
#include <hip/hip_runtime.h>

#define ULLM_DECODE_SCRATCH_FLOATS (2 * 1024 * 1024)
#define ULLM_ERR_SCRATCH (-4)

#ifdef __cplusplus
extern "C" {
#endif

// Floats of scratch the static entry point holds per GPU.  Also looks up the current device's copy of the
// array, so that a later call under stream capture has nothing left to do but launch.
long long ullm_attention_decode_static_capacity(void);

// Same arguments and result as ullm_attention_decode, without the workspace.
int ullm_attention_decode_static(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* token_list, int n_items, const int* positions, const int* token_entry,
    const int* block_table, int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window,
    int num_splits, int waves, hipStream_t stream);

#ifdef __cplusplus
}
#endif
