// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, and harnesses that forbid hipMalloc.
//
// xr_sample_static is xr_sample with the work area of the greedy rows' first pass (a row's
// logits are read by 32 workgroups, each leaving the maximum of its range) in a device array
// that belongs to the library, XR_SAMPLE_STATIC_MAX_ROWS x 32 x 2 floats = 256 KB on every GPU
// the library runs on, held until the process ends.  The caller still passes the logits, the
// per-row options and the output.  It calls no hipMalloc, hipFree or allocating library routine.
// More rows than XR_SAMPLE_STATIC_MAX_ROWS are refused with an error text.
//
// Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two
// threads) race on it and must be ordered by the caller.  The array keeps the last call's
// contents; nothing in it has to start at zero, since the first pass writes every entry that
// the second pass reads.
//
// xr_sample_static_init resolves the array's address on the current device (once per device)
// and may be called at set-up, before a stream is captured; the entry point does the same at
// its first call on a device.
#pragma once

#include "common.h"

#define XR_SAMPLE_STATIC_MAX_ROWS 1024

extern "C" int xr_sample_static_init();
extern "C" int xr_sample_static(int* out, float* logits, int W, int V, int ld, const float* temp, const int* top_k,
                                const float* top_p, const float* min_p, const float* repeat_penalty,
                                const float* draw, const int* recent, const int* n_recent, int recent_cap,
                                const int* exempt, int n_exempt, hipStream_t stream);
