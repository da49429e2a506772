// Entry points for callers that cannot allocate device memory.
//
// llmlab_argmax_static has no counterpart in the reference.  It is for callers
// that must not call hipMalloc: code under HIP graph capture, tight serving loops,
// harnesses that forbid allocation.  It does what llmlab_argmax does (greedy token
// per row of float32 logits, ties to the smallest index, a row of nothing but NaN
// gives -1) with the same two kernels, but the partial maxima of the first stage
// live in a file-scope device array of the library instead of a workspace that the
// caller brings.  The caller still passes the logits and the output.
//
// Limits: rows * ceil(vocab / 8192) <= LLMLAB_ARGMAX_STATIC_PAIRS (each pair is a
// float and an int: the array is 2 * 4 * LLMLAB_ARGMAX_STATIC_PAIRS bytes = 256 KB,
// held on every GPU the library runs on until the process ends).  Larger problems
// are refused with an error; nothing is launched then.
//
// Every call on a GPU uses that GPU's one array, which keeps the contents of the
// last call.  Nothing in it has to start at zero: the first stage writes every
// entry that the second stage reads.  Calls that overlap on one GPU (two streams,
// two threads) race on the array; callers serialise them.
#pragma once

#include <hip/hip_runtime.h>

#define LLMLAB_ARGMAX_STATIC_PAIRS 32768

extern "C" int llmlab_argmax_static(const float* logits, long row_stride, int rows, int vocab,
                                    int* out, hipStream_t stream);
