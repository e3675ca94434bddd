// What the bfloat16 attention kernels share: the head size of the build, fragment types and the few
// one-instruction helpers.  One head size per build (-DHEAD_DIM=N, a multiple of 16 up to 256).
#pragma once
#include "common.hpp"

#ifndef HEAD_DIM
#error "build with -DHEAD_DIM=<multiple of 16>"
#endif
#if HEAD_DIM % 16 != 0 || HEAD_DIM < 16 || HEAD_DIM > 256
#error "HEAD_DIM must be a multiple of 16 from 16 to 256"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = HEAD_DIM;
constexpr int KS = (D + 31) / 32;      // 32-dim steps of q . k
constexpr int DT = D / 16;             // 16-dim tiles of the output
constexpr int BLOCK_KEYS = 32;

union Frag {
  bf16x8 v;
  uint4 q;
  uint2 h[2];
  uint32_t w[4];
};

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

// two floats to two bfloat16 (round to nearest even, one v_cvt_pk_bf16_f32), low half = a
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  const float2_t f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

// max of two numbers neither of which is a NaN, as one instruction (fmaxf adds two more to quiet NaNs)
__device__ __forceinline__ float max_nn(float a, float b) { return __builtin_amdgcn_fmed3f(a, b, INFINITY); }

// max / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one query's or head's lanes), by the lane
// swaps of gfx950 instead of a trip through the LDS: v_permlane16_swap exchanges the odd 16-lane rows of
// its first operand with the even rows of its second, v_permlane32_swap the upper half of the first with
// the lower half of the second; with both operands equal, the pair holds x[l] and x[l ^ 16] (x[l ^ 32]).
__device__ __forceinline__ float quad_max(float x) {      // no NaN among the values
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = max_nn(__uint_as_float(r[0]), __uint_as_float(r[1]));
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return max_nn(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float quad_sum(float x) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// 2^x by the hardware instruction alone: results below 2^-126 are flushed to 0, which a softmax weight may be
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

