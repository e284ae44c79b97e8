// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops, harnesses
// that forbid hipMalloc.  hfee_argmax spreads a row over several workgroups only when
// its caller brings a buffer for their partial results and counters that are zero;
// hfee_argmax_static does the same with a buffer that the library itself holds in a
// file-scope __device__ array, so the caller passes the logits and the output alone.
//
// Limits: at most HFEE_ARGMAX_STATIC_MAX_ROWS rows a call (more are refused with an
// error); the array takes HFEE_ARGMAX_STATIC_BYTES of each GPU that the library runs on,
// until the process ends.  Every call on a GPU shares that GPU's array: calls that
// overlap on one GPU (two streams, two threads) race; calls on one stream do not.
// The first call on a device looks the array's address up (no allocation, but not
// something to do under capture: call once before capturing).
#pragma once
#include "common.h"

#define HFEE_ARGMAX_STATIC_MAX_ROWS 256
#define HFEE_ARGMAX_STATIC_PARTS 64
// per row: PARTS pairs (value, id) of partial results, then one counter a row
#define HFEE_ARGMAX_STATIC_BYTES (HFEE_ARGMAX_STATIC_MAX_ROWS * (HFEE_ARGMAX_STATIC_PARTS * 8 + 4))

// out[r] = id of the first maximum of logits[r * ld .. r * ld + V - 1] (float32), as
// hfee_argmax gives it.  0 on success; else hfee_last_error() has the reason.
HFEE_API int hfee_argmax_static(int* out, const float* logits, int64_t ld, int rows, int V, hipStream_t stream);
