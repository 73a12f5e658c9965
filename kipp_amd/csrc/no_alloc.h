// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// kipp_argmax (sampling.hip) finds the largest logit of every row in two stages when the
// vocabulary is large, and takes a scratch buffer for the partial results of the first stage
// from its caller.  kipp_argmax_static does the same work with the same kernels, and gives
// the same tokens, but keeps those partial results in a device array of fixed size that the
// library itself holds (KIPP_ARGMAX_STATIC_MAX_ROWS * 256 bytes on every GPU the library runs
// on, until the process ends).  It calls no hipMalloc, no hipFree and no allocating library
// routine; the caller still passes the logits and the output.
//
//   logits  float32 [rows, vocab] on the current device
//   out     int32 [rows] on the current device
//   rows    at most KIPP_ARGMAX_STATIC_MAX_ROWS, else the call returns -2 and launches nothing
//   stream  the stream to launch on
//   returns 0, or a negative code for refused arguments, or the HIP error of the launch
//
// All calls on one GPU share that GPU's array.  A call overwrites every slot it reads before it
// reads it, so calls in stream order need no clearing in between; calls that overlap on one
// GPU (two streams, two threads) race on the array and must not be made.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define KIPP_ARGMAX_STATIC_MAX_ROWS 256

extern "C" int kipp_argmax_static_max_rows(void);
extern "C" int kipp_argmax_static(const float* logits, int32_t* out, int rows, int vocab, hipStream_t stream);
