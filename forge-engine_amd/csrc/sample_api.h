// C interface of the sampling library (sample.hip).  Every entry point returns FE_OK,
// FE_BAD_ARGUMENT or FE_LAUNCH_FAILED and launches on the given stream of the current device.
#pragma once
#include <hip/hip_runtime.h>

// Most rows that fe_argmax_rows_static takes in one call.
#define FE_ARGMAX_STATIC_MAX_ROWS 1024

// Four-byte words of parameters that fe_sample_filtered_rows reads per row.
#define FE_SAMPLE_PARAM_WORDS 8

// Most slices (blocks) that fe_sample_filtered_rows cuts a row into, the scratch it needs per row,
// and the launches that rows need at most: the maximum, the sums and the pick, and up to four
// histograms for each of top-k and top-p that any row asks for.
#define FE_SAMPLE_MAX_SPLIT 32
#define FE_SAMPLE_SCRATCH_BYTES_PER_ROW 76800
#define FE_SAMPLE_LAUNCHES(any_top_k, any_top_p) (3 + ((any_top_k) ? 4 : 0) + ((any_top_p) ? 4 : 0))

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
// current.  That first call on a device is set-up: the lookup may make the runtime load the
// library's device image, so it must be made outside any graph capture (one row suffices); every
// later call on that device may be captured.  The call allocates nothing and frees nothing.  rows > FE_ARGMAX_STATIC_MAX_ROWS is
// refused with FE_BAD_ARGUMENT.  Nothing in the array has to start at zero: every word that the
// merge reads is written by the same call first.  All calls on one GPU share the array, so two
// calls that overlap on one GPU (different streams, or threads) race; calls on one stream do not.
int fe_argmax_rows_static(const float* logits, long long row_stride, int rows, int vocab, int* tokens,
                          int* status, hipStream_t stream);

// Rows with parameters of their own.  params: rows x FE_SAMPLE_PARAM_WORDS four-byte words, 8-byte
// aligned: temperature (float; 0 asks for the arg-max), top_k (int; 0 = no limit), top_p (float;
// >= 1 = no limit), min_p (float; 0 = no limit), seed (64 bits), draw index (64 bits).
// tokens[r] is drawn from softmax(logits[r] / temperature) restricted, in this order, to the top_k
// largest entries (with every entry equal to the k-th), to the entries before which at most top_p
// of that set's probability lies, and to those with at least min_p of the largest probability; the
// first kept token, in token order, whose running probability exceeds the uniform
// philox(counter = draw index, key = seed) is taken.  Status bits as for fe_argmax_rows, judged on
// the logits before any filter; bit 3 (8): the launches did not suffice for the row (never, with
// FE_SAMPLE_LAUNCHES of the filters in use).  Probabilities are summed as 64-bit integers (2^-40 of
// the largest one's), so the result does not depend on the order of the sums.
// A row is cut into `split` slices (1 .. FE_SAMPLE_MAX_SPLIT), a block each, and every pass over the
// rows is a launch: `launches` of them.  scratch: rows * FE_SAMPLE_SCRATCH_BYTES_PER_ROW bytes of
// device memory, 8-byte aligned, that the caller owns; it may hold anything.
int fe_sample_filtered_rows(const float* logits, long long row_stride, int rows, int vocab, const void* params,
                            int* tokens, int* status, void* scratch, int split, int launches, hipStream_t stream);

}  // extern "C"
