// Exported entry points of sampling.hip (C linkage; see common.h for the conventions).
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// One token per row of float logits [n_rows, V]: greedy where temperature is null or <= 0 (the
// lowest index among the maxima), else a draw from softmax(logits / temperature[r]) keyed by
// keys[r].  `scratch` is a workspace of jv_sample_scratch_bytes(n_rows) bytes of device memory.
// A row without any comparable value (all NaN) is answered with V.
long long jv_sample_scratch_bytes(int n_rows);
int jv_sample(int* out, const float* logits, long long row_stride, int n_rows, int V, const float* temperature,
              const unsigned long long* keys, void* scratch, void* stream);

// jv_sample for callers that cannot allocate device memory and so have no workspace to pass:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
// counterpart in the reference, which leaves such buffers to its compiler.  The workspace is a
// fixed array inside the library (512 KiB on every GPU the library runs on, kept until the process
// ends), so at most JV_SAMPLE_NOALLOC_MAX_ROWS rows per call: more are refused with
// hipErrorInvalidValue (1) and a sentence in jv_sample_noalloc_last_error() (per thread; empty
// after a call that succeeded).  Neither this call nor jv_sample_noalloc_init allocates or frees
// anything.  Same results as jv_sample, bit for bit.  All calls on one GPU share the array and it
// keeps the last call's contents (every entry that is read is written first, nothing relies on
// zeros): calls that overlap on one GPU race, calls in stream order do not.
// jv_sample_noalloc_init looks up the array's address on the current device; calling it is
// optional (the first call on a device does the same) but keeps that lookup out of a timed or
// captured region.
#define JV_SAMPLE_NOALLOC_MAX_ROWS 1024
int jv_sample_noalloc_init(void);
int jv_sample_noalloc(int* out, const float* logits, long long row_stride, int n_rows, int V,
                      const float* temperature, const unsigned long long* keys, void* stream);
const char* jv_sample_noalloc_last_error(void);

#ifdef __cplusplus
}
#endif
