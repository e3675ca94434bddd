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

// The same from the projection's float32 sums, for steps of many tokens (bfloat16 caches): q and k are
// rounded once, after the rotation.  sums [tokens, ld] float32 (q heads, k heads, v heads); q_out [tokens, ldq]
// bfloat16 gets the rotated q; rotated k and v go to their slots.  Rotation over the whole head.
// grid (ceil(tokens / 16), ceil(heads / 4)): a workgroup takes 16 tokens of 4 heads.  Rotary heads: a thread
// takes four pairs (16 bytes of sums on each side).  Value heads are turned in the LDS ([dim][token]), so that
// a thread owns one dim's 16 tokens: where the 16 tokens are one run of 16
// slots of one page starting at a multiple of 16 (a prompt written from a page's start), they go out as 32
// contiguous bytes; otherwise one by one.
constexpr int RS_TOK = 16, RS_HEADS = 4, RS_VROW = RS_TOK + 8;      // LDS row of a dim: 16 tokens + padding (bf16)

__device__ __forceinline__ uint32_t rs_pack(float a, float b) {
  return (uint32_t)__builtin_bit_cast(uint16_t, __float2bfloat16(a)) | ((uint32_t)__builtin_bit_cast(uint16_t, __float2bfloat16(b)) << 16);
}

__global__ void __launch_bounds__(256)
rotary_kv_store_sums_kernel(const float* __restrict__ sums, long ld, bf16* __restrict__ q_out, long ldq,
                            const int* __restrict__ positions, const float* __restrict__ cos_t,
                            const float* __restrict__ sin_t, const int* __restrict__ slots, bf16* __restrict__ k_cache,
                            bf16* __restrict__ v_cache, int Hq, int Hkv, int D, int page, int tokens) {
  extern __shared__ __align__(16) unsigned char rs_lds[];
  __shared__ int s_slot[RS_TOK], s_pos[RS_TOK];
  bf16* vt = reinterpret_cast<bf16*>(rs_lds);                       // [RS_HEADS * D][RS_VROW]
  const int t0 = blockIdx.x * RS_TOK, n = tokens - t0 < RS_TOK ? tokens - t0 : RS_TOK;
  const int h0 = blockIdx.y * RS_HEADS, heads = Hq + 2 * Hkv;
  const int nh = heads - h0 < RS_HEADS ? heads - h0 : RS_HEADS;
  if (threadIdx.x < RS_TOK) {
    const int t = t0 + (threadIdx.x < n ? threadIdx.x : 0);
    s_slot[threadIdx.x] = slots[t];
    s_pos[threadIdx.x] = positions[t];
  }
  __syncthreads();
  const int half = D >> 1, groups = half >> 2;                      // four pairs a thread
  // ---- q and k heads of this chunk
  const int rot_heads = h0 >= Hq + Hkv ? 0 : (Hq + Hkv - h0 < nh ? Hq + Hkv - h0 : nh);
  for (int w = threadIdx.x; w < n * rot_heads * groups; w += blockDim.x) {
    const int jg = w % groups, rest = w / groups, hh = rest % rot_heads, i = rest / rot_heads;
    const int head = h0 + hh, j = jg << 2, t = t0 + i;
    const float* src = sums + (size_t)t * ld + (size_t)head * D;
    const float4 a = *reinterpret_cast<const float4*>(src + j), b = *reinterpret_cast<const float4*>(src + j + half);
    const float4 c = *reinterpret_cast<const float4*>(cos_t + (size_t)s_pos[i] * half + j);
    const float4 sn = *reinterpret_cast<const float4*>(sin_t + (size_t)s_pos[i] * half + j);
    float r1[4], r2[4];
    rotate_pair(a.x, b.x, c.x, sn.x, r1[0], r2[0]);
    rotate_pair(a.y, b.y, c.y, sn.y, r1[1], r2[1]);
    rotate_pair(a.z, b.z, c.z, sn.z, r1[2], r2[2]);
    rotate_pair(a.w, b.w, c.w, sn.w, r1[3], r2[3]);
    uint2 o1, o2;
    o1.x = rs_pack(r1[0], r1[1]);
    o1.y = rs_pack(r1[2], r1[3]);
    o2.x = rs_pack(r2[0], r2[1]);
    o2.y = rs_pack(r2[2], r2[3]);
    bf16* dst;
    if (head < Hq) {
      dst = q_out + (size_t)t * ldq + (size_t)head * D;
    } else {
      const int slot = s_slot[i];
      dst = k_cache + (((size_t)(slot / page) * Hkv + (head - Hq)) * page + (size_t)(slot % page)) * D;
    }
    *reinterpret_cast<uint2*>(dst + j) = o1;
    *reinterpret_cast<uint2*>(dst + j + half) = o2;
  }
  // ---- v heads of this chunk (the condition is the same for the whole workgroup)
  const int v_first = h0 > Hq + Hkv ? h0 : Hq + Hkv;                // first value head of this chunk
  const int v_heads = h0 + nh - v_first;
  if (v_heads <= 0) return;
  const int d4 = D >> 2;
  for (int w = threadIdx.x; w < n * v_heads * d4; w += blockDim.x) {
    const int dg = w % d4, rest = w / d4, hh = rest % v_heads, i = rest / v_heads;
    const float4 a = *reinterpret_cast<const float4*>(sums + (size_t)(t0 + i) * ld + (size_t)(v_first + hh) * D + dg * 4);
    bf16* at = vt + (size_t)(hh * D + dg * 4) * RS_VROW + i;
    at[0] = __float2bfloat16(a.x);
    at[RS_VROW] = __float2bfloat16(a.y);
    at[2 * RS_VROW] = __float2bfloat16(a.z);
    at[3 * RS_VROW] = __float2bfloat16(a.w);
  }
  __syncthreads();
  bool run = n == RS_TOK && (s_slot[0] & 15) == 0 && s_slot[0] % page + RS_TOK <= page;
  for (int i = 1; i < RS_TOK; ++i) run = run && s_slot[i] == s_slot[0] + i;
  for (int w = threadIdx.x; w < v_heads * D; w += blockDim.x) {
    const int hh = w / D, d = w - hh * D, kvh = v_first + hh - Hq - Hkv;
    const bf16* from = vt + (size_t)w * RS_VROW;
    if (run) {
      bf16* dst = v_cache + (((size_t)(s_slot[0] / page) * Hkv + kvh) * D + d) * page + (size_t)(s_slot[0] % page);
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(from);
      *reinterpret_cast<uint4*>(dst + 8) = *reinterpret_cast<const uint4*>(from + 8);
    } else {
      for (int i = 0; i < n; ++i) {
        const int slot = s_slot[i];
        v_cache[(((size_t)(slot / page) * Hkv + kvh) * D + d) * page + (size_t)(slot % page)] = from[i];
      }
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

// sums [tokens, ld] float32, the q/k/v projection before rounding; bfloat16 q_out and caches; head_dim a
// multiple of 8, rotation over the whole head.
MIE_EXPORT int mie_rotary_kv_store_sums(const float* sums, long ld, void* q_out, long ldq, const int* positions,
                                        const float* cos_t, const float* sin_t, const int* slots, void* k_cache,
                                        void* v_cache, int Hq, int Hkv, int D, int page, int tokens, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (D <= 0 || (D & 7)) MIE_FAIL("rotary_kv_store_sums: head_dim %d must be a multiple of 8", D);
  if (Hq <= 0 || Hkv <= 0 || page < 16 || (page & 15)) MIE_FAIL("rotary_kv_store_sums: heads %d / %d, page %d", Hq, Hkv, page);
  if (!sums || !q_out || !positions || !cos_t || !sin_t || !slots || !k_cache || !v_cache) MIE_FAIL("rotary_kv_store_sums: null operand");
  if (ld < (long)(Hq + 2 * Hkv) * D || (ld & 3) || ldq < (long)Hq * D || (ldq & 3)) MIE_FAIL("rotary_kv_store_sums: leading dims %ld, %ld", ld, ldq);
  if ((((uintptr_t)sums | (uintptr_t)cos_t | (uintptr_t)sin_t | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) || ((uintptr_t)q_out & 7))
    MIE_FAIL("rotary_kv_store_sums: operands must be 16-byte aligned");
  const int lds_bytes = RS_HEADS * D * RS_VROW * (int)sizeof(bf16);
  if (lds_bytes > 64 * 1024) MIE_FAIL("rotary_kv_store_sums: head_dim %d needs %d bytes of LDS", D, lds_bytes);
  dim3 grid((tokens + RS_TOK - 1) / RS_TOK, (Hq + 2 * Hkv + RS_HEADS - 1) / RS_HEADS);
  hipLaunchKernelGGL(rotary_kv_store_sums_kernel, grid, dim3(256), lds_bytes, stream, sums, ld, (bf16*)q_out, ldq, positions, cos_t,
                     sin_t, slots, (bf16*)k_cache, (bf16*)v_cache, Hq, Hkv, D, page, tokens);
  MIE_CHECK_LAUNCH("rotary_kv_store_sums");
  return 0;
}
