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
  else if (dtype == MIE_BF16)
    hipLaunchKernelGGL(rotary_kv_store_kernel<bf16>, grid, block, 0, stream, (bf16*)qkv, row_stride, positions, cos_t,
                       sin_t, rot, Hq, Hkv, D, (bf16*)k_cache, (bf16*)v_cache, slots, page);
  else
    MIE_FAIL("rotary_kv_store: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("rotary_kv_store");
  return 0;
}
