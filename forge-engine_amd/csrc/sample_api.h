// C interface of the sampling library (sample.hip).  Every entry point returns FE_OK,
// FE_BAD_ARGUMENT or FE_LAUNCH_FAILED and launches on the given stream of the current device.
#pragma once
#include <hip/hip_runtime.h>

// Most rows that fe_argmax_rows_static takes in one call.
#define FE_ARGMAX_STATIC_MAX_ROWS 1024

extern "C" {

// tokens[r] = argmax(logits[r]) (lowest index among equals); status bits: 1 NaN, 2 +inf, 4 no finite
// entry.  scratch: at least rows * 32 * 3 four-byte words of device memory that the caller owns.
int fe_argmax_rows(const float* logits, long long row_stride, int rows, int vocab, int* tokens, int* status,
                   void* scratch, hipStream_t stream);

// The same result as fe_argmax_rows (the same two kernels) for callers that cannot allocate
// device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  It has no counterpart in the reference, whose sampling goes through torch's
// allocator.  The partial maxima live in an array inside the library's device image
// (FE_ARGMAX_STATIC_MAX_ROWS * 32 * 3 words = 384 KiB on each GPU the library runs on, until the
// process ends); its address on a device is looked up once, at the first call with that device
// current.  The call allocates nothing and frees nothing.  rows > FE_ARGMAX_STATIC_MAX_ROWS is
// refused with FE_BAD_ARGUMENT.  Nothing in the array has to start at zero: every word that the
// merge reads is written by the same call first.  All calls on one GPU share the array, so two
// calls that overlap on one GPU (different streams, or threads) race; calls on one stream do not.
int fe_argmax_rows_static(const float* logits, long long row_stride, int rows, int vocab, int* tokens,
                          int* status, hipStream_t stream);

// tokens[r] drawn from softmax(logits[r] / temperatures[r]) with the uniform
// philox(counter = draw_index[r], key = seeds[r]); entries equal to -inf have probability 0.
int fe_sample_rows(const float* logits, long long row_stride, int rows, int vocab, const float* temperatures,
                   const unsigned long long* seeds, const unsigned long long* draw_index, int* tokens,
                   int* status, hipStream_t stream);

}  // extern "C"
