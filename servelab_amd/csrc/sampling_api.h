// C ABI of the sampling unit (sampling.hip).  Every entry point returns nullptr
// on success or a static message that names the size it refuses; all work is
// queued on `stream`.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

extern "C" {

// Bytes of device scratch that sl_argmax / sl_sample need for R rows cut into
// `chunks` slices (`cuts`: some row has a top-k or top-p cut).
size_t sl_sample_workspace(int R, int chunks, int cuts);

// out[r] = index of the largest of logits[r, 0..V) (ties: the first).
const char* sl_argmax(const float* logits, int R, int V, int chunks, void* work, int* out,
                      hipStream_t stream);

// One token per row: greedy where temperature[r] == 0 (or temperature == nullptr),
// else a draw from softmax(logits / T), optionally cut by top_k / top_p.
const char* sl_sample(const float* logits, int R, int V, const float* temperature,
                      const int* top_k, const float* top_p, const int64_t* seeds,
                      const int64_t* draws, int chunks, void* work, int* out, hipStream_t stream);

// sl_sample for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
// no counterpart in the reference.  Same arguments and results as sl_sample,
// but the scratch is a static device array of SL_SAMPLE_STATIC_BYTES inside the
// library (each GPU the library runs on holds its own copy until the process
// ends) and the split of a row into slices is chosen here.  Sizes whose scratch
// would not fit are refused with a message.  The call allocates and frees
// nothing.  All calls on one GPU share that GPU's array: calls that overlap on
// one GPU (two streams, two threads) race; calls on one stream do not.  Nothing
// in the array has to start at zero, since every stage of a call writes all that
// the next stage reads, so it is never cleared.
#define SL_SAMPLE_STATIC_BYTES (8u << 20)
const char* sl_sample_static(const float* logits, int R, int V, const float* temperature,
                             const int* top_k, const float* top_p, const int64_t* seeds,
                             const int64_t* draws, int* out, hipStream_t stream);

}  // extern "C"
