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
