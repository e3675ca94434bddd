// Decode attention for callers that cannot allocate.
//
// This entry point has no counterpart in the reference.  It exists for callers that may not call
// hipMalloc (directly or through torch): code under HIP graph capture, tight serving loops, harnesses
// that forbid allocation.  It computes exactly what mie_decode_attention computes, with the same kernels;
// the only difference is where the partial results of a split context live.  mie_decode_attention takes
// them from the caller (o_part, lse_part); this one keeps them in an array in the library's own device
// image, so it calls no hipMalloc, no hipFree and no allocating library routine.
//
// The array is MIE_DECODE_STATIC_SCRATCH_BYTES large and exists once on every GPU the library is used
// on, until the process ends.  A call needs rows * Hq * num_splits * (head_dim + 1) floats of it and is
// refused with a message if that is more.  Every call on a GPU uses that GPU's one array: calls that
// overlap on one GPU (two streams, two threads) race on it; calls on one stream do not.  Nothing in it
// has to start at zero: each call writes every log-sum-exp it later reads, and a partial result is read
// only where its log-sum-exp is finite.
//
// mie_decode_attention_static_setup() looks the array's device address up for the current device and
// keeps it; the first call of the entry point on a device does the same if set-up was not called.  A
// caller that records graphs calls set-up once per device before it starts recording.
#pragma once
#include <hip/hip_runtime.h>

#ifndef MIE_EXPORT
#define MIE_EXPORT extern "C" __attribute__((visibility("default")))
#endif

#define MIE_DECODE_STATIC_SCRATCH_BYTES (8u << 20)

// 0, or -1 with a message in attention_bf16_last_error()
MIE_EXPORT int mie_decode_attention_static_setup(void);

// the array's size in bytes
MIE_EXPORT long mie_decode_attention_static_capacity(void);

// Arguments as mie_decode_attention without o_part and lse_part.
MIE_EXPORT int mie_decode_attention_static(const void* q, long q_stride, const void* k_cache, const void* v_cache,
                                           void* out, const int* block_tables, int max_blocks, const int* positions,
                                           int rows, int Hq, int Hkv, int head_dim, int page, float scale, int window,
                                           int partition, int num_splits, hipStream_t stream);
