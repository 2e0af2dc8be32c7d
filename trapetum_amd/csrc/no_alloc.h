// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops that must not reach hipMalloc, harnesses that forbid it.  The caller passes
// inputs and outputs as for tp_argmax; what tp_argmax takes as a workspace argument lives in a fixed device array
// inside the library instead.
#pragma once

// rows one call takes, parts a row is scanned in, and the size of the fixed array (a float and an int per row and part)
#define TP_ARGMAX_NO_ALLOC_MAX_ROWS 256
#define TP_ARGMAX_NO_ALLOC_PARTS 64
#define TP_ARGMAX_NO_ALLOC_SCRATCH_BYTES (TP_ARGMAX_NO_ALLOC_MAX_ROWS * TP_ARGMAX_NO_ALLOC_PARTS * 8)

#ifdef __cplusplus
extern "C" {
#endif

// out[b] = the smallest index among the largest values of logits[b, 0 .. V) (float32, rows V apart; NaN never wins),
// the result tp_argmax gives.  B up to TP_ARGMAX_NO_ALLOC_MAX_ROWS, any V > 0; more rows are refused with an error
// (non-zero return, text from tp_last_error()).  Enqueued on `stream` (a hipStream_t); calls no hipMalloc, hipFree or
// allocating library routine.  Each GPU holds one scratch array of TP_ARGMAX_NO_ALLOC_SCRATCH_BYTES that every call
// on that GPU shares: calls that overlap on one GPU race; calls in stream order do not.
// The first call on a device also asks the runtime where that device's copy of the array lies, which is no stream
// operation (it may load the library's code on that device): make that first call, or tp_argmax_no_alloc_prepare(),
// outside any stream capture; every later call on the device only enqueues two kernels and may be captured.
int tp_argmax_no_alloc(const float* logits, int B, int V, int* out, void* stream);

// Resolves the scratch array's address on the current device and launches nothing: for callers that want the first
// tp_argmax_no_alloc on a device to be inside a stream capture.  Returns 0, or non-zero with a message.
int tp_argmax_no_alloc_prepare(void);

#ifdef __cplusplus
}
#endif
