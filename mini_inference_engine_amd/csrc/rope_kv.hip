// Rotary position encoding (half-split pairs) of q and k inside the fused projection output,
// fused with the write of k and v into their cache slots.
//
// qkv row t: [ q heads (Hq * D) | k heads (Hkv * D) | v heads (Hkv * D) ], row stride given.
// For every q and k head and j < rot / 2, with c, s = cos, sin[position[t], j] (32-bit tables):
//   out[j]           = x[j] c - x[j + rot/2] s
//   out[j + rot/2]   = x[j + rot/2] c + x[j] s            (computed in 32-bit, rounded once)
// dims rot..D of a head are left as they are.  k (rotated) and v of token t go to slot
// slot_mapping[t]: keys into a cache laid out [pages, Hkv, page, D], values into one laid out
// [pages, Hkv, D, page] (a page's values transposed: the 16+ keys of one dim are contiguous,
// which is how the attention kernels' matrix instructions want them).
#include "common.hpp"

template <typename T>
__global__ void __launch_bounds__(256)
rotary_kv_store_kernel(T* __restrict__ qkv, long row_stride, const int* __restrict__ positions,
                       const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int Hq, int Hkv,
                       int D, T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ slots,
                       int page) {
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * row_stride;
  const int half = rot >> 1;
  size_t k_base = 0, v_base = 0;
  if (Hkv) {
    const int slot = slots[t];
    k_base = ((size_t)(slot / page) * Hkv * page + (size_t)(slot % page)) * D;   // + kvh * page * D
    v_base = (size_t)(slot / page) * Hkv * page * D + (size_t)(slot % page);     // + (kvh * D + d) * page
  }
  if (half) {
    const int pos = positions[t];
    const float* cr = cos_t + (size_t)pos * half;
    const float* sr = sin_t + (size_t)pos * half;
    const int pairs = (Hq + Hkv) * half;
    for (int w = threadIdx.x; w < pairs; w += blockDim.x) {
      const int head = w / half, j = w - head * half;
      T* hp = row + (size_t)head * D;
      const float x1 = to_float(hp[j]), x2 = to_float(hp[j + half]);
      const float c = cr[j], s = sr[j];
      const T o1 = from_float<T>(x1 * c - x2 * s), o2 = from_float<T>(x2 * c + x1 * s);
      hp[j] = o1;
      hp[j + half] = o2;
      if (head >= Hq) {
        T* kc = k_cache + k_base + (size_t)(head - Hq) * page * D;
        kc[j] = o1;
        kc[j + half] = o2;
      }
    }
  }
  if (Hkv) {
    // unrotated tail of k, and all of v
    const int tail = D - rot;
    for (int w = threadIdx.x; w < Hkv * tail; w += blockDim.x) {
      const int kvh = w / tail, d = rot + (w - kvh * tail);
      k_cache[k_base + (size_t)kvh * page * D + d] = row[(size_t)(Hq + kvh) * D + d];
    }
    for (int w = threadIdx.x; w < Hkv * D; w += blockDim.x) {
      const int kvh = w / D, d = w - kvh * D;
      v_cache[v_base + ((size_t)kvh * D + d) * page] = row[(size_t)(Hq + Hkv + kvh) * D + d];
    }
  }
}

// bfloat16, rotary_dim a multiple of 16, rows and cache on 16 bytes: a thread takes eight pairs (j .. j + 7 and
// their partners), so rows move 16 bytes a load.  The unrotated tail of k (if any) and v go as in the kernel above.
__global__ void __launch_bounds__(256)
rotary_kv_store_bf16x8_kernel(bf16* __restrict__ qkv, long row_stride, const int* __restrict__ positions,
                              const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int Hq, int Hkv,
                              int D, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
                              const int* __restrict__ slots, int page) {
  const int t = blockIdx.x;
  bf16* row = qkv + (size_t)t * row_stride;
  const int half = rot >> 1, groups = half >> 3;
  size_t k_base = 0, v_base = 0;
  if (Hkv) {
    const int slot = slots[t];
    k_base = ((size_t)(slot / page) * Hkv * page + (size_t)(slot % page)) * D;
    v_base = (size_t)(slot / page) * Hkv * page * D + (size_t)(slot % page);
  }
  const int pos = positions[t];
  const float* cr = cos_t + (size_t)pos * half;
  const float* sr = sin_t + (size_t)pos * half;
  for (int w = threadIdx.x; w < (Hq + Hkv) * groups; w += blockDim.x) {
    const int head = w / groups, j = (w - head * groups) << 3;
    bf16* hp = row + (size_t)head * D;
    const uint4 a4 = *reinterpret_cast<const uint4*>(hp + j), b4 = *reinterpret_cast<const uint4*>(hp + j + half);
    const float4 c0 = *reinterpret_cast<const float4*>(cr + j), c1 = *reinterpret_cast<const float4*>(cr + j + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(sr + j), s1 = *reinterpret_cast<const float4*>(sr + j + 4);
    const uint32_t aw[4] = {a4.x, a4.y, a4.z, a4.w}, bw[4] = {b4.x, b4.y, b4.z, b4.w};
    const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    uint32_t o1[4], o2[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float x1l = __uint_as_float(aw[e] << 16), x1h = __uint_as_float(aw[e] & 0xFFFF0000u);
      const float x2l = __uint_as_float(bw[e] << 16), x2h = __uint_as_float(bw[e] & 0xFFFF0000u);
      const bf16 r1l = __float2bfloat16(x1l * c[2 * e] - x2l * sn[2 * e]);
      const bf16 r1h = __float2bfloat16(x1h * c[2 * e + 1] - x2h * sn[2 * e + 1]);
      const bf16 r2l = __float2bfloat16(x2l * c[2 * e] + x1l * sn[2 * e]);
      const bf16 r2h = __float2bfloat16(x2h * c[2 * e + 1] + x1h * sn[2 * e + 1]);
      o1[e] = (uint32_t)__builtin_bit_cast(uint16_t, r1l) | ((uint32_t)__builtin_bit_cast(uint16_t, r1h) << 16);
      o2[e] = (uint32_t)__builtin_bit_cast(uint16_t, r2l) | ((uint32_t)__builtin_bit_cast(uint16_t, r2h) << 16);
    }
    const uint4 v1 = make_uint4(o1[0], o1[1], o1[2], o1[3]), v2 = make_uint4(o2[0], o2[1], o2[2], o2[3]);
    *reinterpret_cast<uint4*>(hp + j) = v1;
    *reinterpret_cast<uint4*>(hp + j + half) = v2;
    if (head >= Hq) {
      bf16* kc = k_cache + k_base + (size_t)(head - Hq) * page * D;
      *reinterpret_cast<uint4*>(kc + j) = v1;
      *reinterpret_cast<uint4*>(kc + j + half) = v2;
    }
  }
  if (Hkv) {
    const int tail = D - rot;
    for (int w = threadIdx.x; w < Hkv * tail; w += blockDim.x) {
      const int kvh = w / tail, d = rot + (w - kvh * tail);
      k_cache[k_base + (size_t)kvh * page * D + d] = row[(size_t)(Hq + kvh) * D + d];
    }
    for (int w = threadIdx.x; w < Hkv * D; w += blockDim.x) {
      const int kvh = w / D, d = w - kvh * D;
      v_cache[v_base + ((size_t)kvh * D + d) * page] = row[(size_t)(Hq + Hkv + kvh) * D + d];
    }
  }
}

MIE_EXPORT const char* rope_kv_last_error() { return g_mie_error; }

MIE_EXPORT int mie_rotary_kv_store(void* qkv, int dtype, long row_stride, const int* positions, const float* cos_t,
                                   const float* sin_t, int rot, int Hq, int Hkv, int D, void* k_cache, void* v_cache,
                                   const int* slots, int page, int tokens, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (rot < 0 || rot > D || (rot & 1)) MIE_FAIL("rotary_kv_store: rotary_dim %d with head_dim %d", rot, D);
  if (rot && (!cos_t || !sin_t || !positions)) MIE_FAIL("rotary_kv_store: rotation asked for without tables");
  if (Hkv && (!k_cache || !v_cache || !slots || page <= 0)) MIE_FAIL("rotary_kv_store: cache write asked for without a cache");
  if (row_stride < (long)(Hq + 2 * Hkv) * D) MIE_FAIL("rotary_kv_store: row stride %ld < %d", row_stride, (Hq + 2 * Hkv) * D);
  dim3 grid(tokens), block(256);
  if (dtype == MIE_F32)
    hipLaunchKernelGGL(rotary_kv_store_kernel<float>, grid, block, 0, stream, (float*)qkv, row_stride, positions, cos_t,
                       sin_t, rot, Hq, Hkv, D, (float*)k_cache, (float*)v_cache, slots, page);
  else if (dtype == MIE_BF16 && rot > 0 && (rot & 15) == 0 && (D & 7) == 0 && (row_stride & 7) == 0 &&
           (((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)cos_t | (uintptr_t)sin_t) & 15) == 0)
    hipLaunchKernelGGL(rotary_kv_store_bf16x8_kernel, grid, block, 0, stream, (bf16*)qkv, row_stride, positions, cos_t,
                       sin_t, rot, Hq, Hkv, D, (bf16*)k_cache, (bf16*)v_cache, slots, page);
  else if (dtype == MIE_BF16)
    hipLaunchKernelGGL(rotary_kv_store_kernel<bf16>, grid, block, 0, stream, (bf16*)qkv, row_stride, positions, cos_t,
                       sin_t, rot, Hq, Hkv, D, (bf16*)k_cache, (bf16*)v_cache, slots, page);
  else
    MIE_FAIL("rotary_kv_store: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("rotary_kv_store");
  return 0;
}
