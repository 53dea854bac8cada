// Entry point that allocates nothing.
//
// rl_argmax_static has no counterpart in the reference.  It exists for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops that must never
// reach the allocator, and harnesses that forbid hipMalloc.  It is rl_argmax's two-stage form
// (the best of every slice of a row, then the best of the slices) with the stage-one results in
// a file-scope device array of the library instead of a workspace of the caller.
//
//   * Limit: rows * rl_argmax_slices(vocab) <= RL_ARGMAX_STATIC_ENTRIES (8 bytes each, 128 KB
//     on every GPU the library runs on, held until the process ends).  Beyond it the call
//     returns RL_ERR_ARG and launches nothing.
//   * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
//     streams, two threads) race.  Calls on one stream are ordered and safe.  Nothing has to
//     start at zero: stage one writes every entry that stage two reads.
//   * The array's address is looked up once per device (hipGetSymbolAddress), at the first
//     call on that device or by rl_argmax_static_prepare(), which a caller runs before it
//     starts a capture.  Neither allocates.
#pragma once

#include <hip/hip_runtime.h>

#define RL_ARGMAX_STATIC_ENTRIES 16384
#define RL_ERR_SETUP 3  // the device array's address could not be obtained

extern "C" int rl_argmax_static_prepare();
extern "C" int rl_argmax_static_limit();
extern "C" int rl_argmax_static(const float* logits, const int* row_index, int* out, int rows,
                                int vocab, hipStream_t stream);
