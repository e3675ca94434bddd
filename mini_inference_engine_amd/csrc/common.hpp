// Shared device helpers for the gfx950 kernels: element types, wave reductions,
// launch checking.  Every kernel file exports plain C entry points that take raw
// device pointers and a stream, return 0 or a negative code, and leave a message
// readable through <module>_last_error().
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stdio.h>

#define MIE_WAVE 64

typedef __hip_bfloat16 bf16;

// ---- dtype codes shared with the Python side
enum { MIE_F32 = 0, MIE_BF16 = 1 };

// ---- element conversion (bf16 <-> float); round to nearest even on store
__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16 x) { return __bfloat162float(x); }
template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float x) { return __float2bfloat16(x); }

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// ---- wave-wide reductions (64 lanes), fixed order
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, MIE_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MIE_WAVE));
  return v;
}

// Block-wide sum for blocks of up to 1024 threads; ``scratch`` holds 16 floats.
// Every thread gets the total; the order of additions depends on nothing but blockDim.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += scratch[i];
  return t;
}

// ---- partial sums of a product whose K was split over workgroups
constexpr int MIE_SPLITS_AHEAD = 8;      // splits whose loads are issued together

// acc += the splits' values at p, in split order.  The loads of up to MIE_SPLITS_AHEAD splits are issued
// together, each unconditional from an address clamped to the last split (what it brings for a split that does
// not exist is not added), so a kernel waits for memory once per MIE_SPLITS_AHEAD splits and not once per split.
template <typename V>
__device__ __forceinline__ void add_splits(V& acc, const V* p, int splits, size_t split_stride_v) {
  for (int s0 = 0; s0 < splits; s0 += MIE_SPLITS_AHEAD) {
    V v[MIE_SPLITS_AHEAD];
#pragma unroll
    for (int j = 0; j < MIE_SPLITS_AHEAD; ++j) v[j] = p[(size_t)(s0 + j < splits ? s0 + j : splits - 1) * split_stride_v];
#pragma unroll
    for (int j = 0; j < MIE_SPLITS_AHEAD; ++j)
      if (s0 + j < splits) acc += v[j];
  }
}

// ---- rotary position encoding of one pair, from float32: (x1, x2) turned by the angle whose cosine and sine
// are c and s.  One spelling for every kernel that rotates float32 sums, so that they round alike.
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c, float s, float& o1, float& o2) {
  o1 = fmaf(x1, c, -(x2 * s));
  o2 = fmaf(x2, c, x1 * s);
}

// ---- host-side error plumbing
static thread_local char g_mie_error[512];
#define MIE_FAIL(...)                                        \
  do {                                                       \
    snprintf(g_mie_error, sizeof g_mie_error, __VA_ARGS__);  \
    return -1;                                               \
  } while (0)
#define MIE_CHECK_LAUNCH(name)                                                             \
  do {                                                                                     \
    hipError_t e_ = hipGetLastError();                                                     \
    if (e_ != hipSuccess) MIE_FAIL("%s: launch failed: %s", name, hipGetErrorString(e_));  \
  } while (0)
#define MIE_EXPORT extern "C" __attribute__((visibility("default")))
