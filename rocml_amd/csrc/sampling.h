// Entry points of the sampling library that other native code may call directly.
#pragma once
#include <hip/hip_runtime.h>

// rocml_argmax_static has no counterpart in the reference.  It is rocml_argmax for callers that
// cannot allocate device memory or carry a workspace around: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc.  The partial results of its two stages live in an array of the library
// itself, ROCML_ARGMAX_STATIC_MAX_ROWS * 64 32-bit words (256 KiB) that every GPU the library
// runs on holds until the process ends; the call allocates and frees nothing.
//
//   logits  [batch, vocab] 32-bit floats on the current device
//   out     [batch] 32-bit integers: the first index of each row's maximum
//   batch   at most ROCML_ARGMAX_STATIC_MAX_ROWS, else the call fails (nonzero status, message in
//           sampling_last_error()) and launches nothing
//
// All calls on one GPU share that GPU's array: two calls that overlap in time there (different
// streams, different threads) race and may return each other's partial results; calls on one
// stream, one after the other, are safe.  Nothing in the array has to be zero: every word a
// call reads it has written before.
#define ROCML_ARGMAX_STATIC_MAX_ROWS 1024

extern "C" int rocml_argmax_static(const float* logits, int batch, int vocab, int* out, hipStream_t stream);
