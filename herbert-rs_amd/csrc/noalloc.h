// An entry point that allocates nothing.
//
// It has no counterpart in xigh/herbert-rs. It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// hb_argmax_noalloc is hb_argmax (sampling.hip) without the caller's workspace: the partial
// results of the first stage (one value and one index for every stretch of every row) go
// into an array that the library itself holds in device memory, one copy on every GPU the
// library runs on, from the first call there until the process ends.
//
//   logits  float32 [R, ld], device memory; V <= ld values of a row are looked at
//   out     int32 [R], device memory: the first index of the largest value of each row
//   stream  the stream the two kernels are put on; the device it belongs to must be current
//
// Limit: a row of at least 16384 values is cut into min(64, V / 8192) stretches, and
// R x stretches may not exceed HB_ARGMAX_NOALLOC_MAX_PAIRS; beyond that the call returns
// non-zero without launching anything and hb_last_error() says so (hb_argmax with a workspace
// of the caller's takes any size). Shorter rows take one stretch and no scratch, at any R.
//
// The call allocates nothing and frees nothing (the address of the array is looked up once
// per device, at the first call there or by hb_argmax_noalloc_setup). Every call on a GPU
// shares that GPU's array: calls that overlap in time on one GPU (two streams, two threads)
// race on it; calls on one stream are ordered and safe. Nothing in the array has to start at
// zero: the second kernel reads only what the first has just written.
#pragma once
#include <hip/hip_runtime.h>

#define HB_ARGMAX_NOALLOC_MAX_PAIRS 4096      // 32 KB of device memory per GPU

extern "C" int hb_argmax_noalloc_setup(void);
extern "C" int hb_argmax_noalloc(const float* logits, int ld, int R, int V, int* out, hipStream_t stream);
