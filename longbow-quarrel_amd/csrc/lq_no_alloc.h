// An entry point for callers that cannot allocate device memory.
//
// It has no counterpart in the reference.  Every other entry point of this library takes its scratch
// memory as an argument, which the caller allocates.  Some callers cannot: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  For them the greedy arg-max exists a
// second time with its scratch (the best key of each of 32 slices of every row, which the first stage
// leaves for the second) in a fixed array in device memory that the library itself holds, one copy on
// every GPU it runs on, until the process ends.
#pragma once

#include <hip/hip_runtime.h>

// the most rows one call takes; the array is LQ_ARGMAX_NO_ALLOC_MAX_ROWS * 32 * 8 bytes = 256 KiB a GPU
#define LQ_ARGMAX_NO_ALLOC_MAX_ROWS 1024

// out[r] = first maximal index of logits[r, 0..V) (float32, rows `ld` apart), or -1 for a row that holds
// a NaN or an infinity: what lq_argmax gives without a ring of recent ids.  Allocates nothing and calls
// nothing that does; the device that `stream` belongs to must be current.  Returns 0, or a negative
// code with the reason in lq_last_error(): more than LQ_ARGMAX_NO_ALLOC_MAX_ROWS rows are refused.
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
// threads) race; calls on one stream, or ordered by events, do not.  Nothing in the array has to start
// at zero (the first stage writes every entry that the second reads), so it is never cleared.
// The first call on a device asks the runtime for that device's address of the array (under a lock,
// once): make that call before a stream capture begins, since the query is no stream work and a
// capture may refuse it; every later call on the device only launches the two kernels.
extern "C" int lq_argmax_no_alloc(const float* logits, int ld, int rows, int V, int* out, hipStream_t stream);
