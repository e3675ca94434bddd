// Paged causal attention, one kernel for every kind of row (single decoded tokens and prompt
// portions starting anywhere), in true 32-bit arithmetic for float and bfloat16 storage.
//
// One wavefront per (token, query head).  The token sits in row r at absolute position p and
// sees keys lo..p of its own request, lo = max(0, p - window + 1) or 0, found through the
// row's block table in caches laid out [pages, Hkv, page, D] (keys) and [pages, Hkv, D, page]
// (values, transposed within a page).  Keys are taken 64 at a time
// (one per lane: q . k in increasing d), the softmax is kept online in 32-bit, and the 64
// probabilities then weight the value rows with the lanes spread over D.  The order of every
// sum depends only on (lo, p): the result for a token is bit-identical whatever else the
// step holds and however the request was cut into steps.
//
// This is the reference kernel of the engine: the float32 path runs on it, and the
// bfloat16 path uses it wherever a faster kernel does not take the shape.
#include "common.hpp"

template <typename T> struct Pack;
template <> struct Pack<float> {
  typedef float4 V;
  static constexpr int N = 4;
  __device__ static __forceinline__ void unpack(const V& v, float* f) { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
};
template <> struct Pack<bf16> {
  typedef uint4 V;
  static constexpr int N = 8;
  __device__ static __forceinline__ void unpack(const V& v, float* f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
  }
};

#define ATT_MAX_D 256

template <typename T>
__global__ void __launch_bounds__(64)
paged_attention_kernel(const T* __restrict__ q, long q_stride, const T* __restrict__ k_cache,
                       const T* __restrict__ v_cache, T* __restrict__ out, const int* __restrict__ block_tables,
                       int max_blocks, const int* __restrict__ token_row, const int* __restrict__ positions, int Hq,
                       int Hkv, int D, int page, float scale, int window) {
  __shared__ float qs[ATT_MAX_D];
  __shared__ float ps[64];
  __shared__ long long base[64];     // per key of the chunk: offset of its value column
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int row = token_row[t], pos = positions[t];
  const int kvh = h / (Hq / Hkv);
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int* bt = block_tables + (size_t)row * max_blocks;
  const T* qp = q + (size_t)t * q_stride + (size_t)h * D;
  for (int d = lane; d < D; d += 64) qs[d] = to_float(qp[d]);
  __syncthreads();

  typedef Pack<T> P;
  float m = -INFINITY, l = 0.f;
  float acc[ATT_MAX_D / 64];
#pragma unroll
  for (int i = 0; i < ATT_MAX_D / 64; ++i) acc[i] = 0.f;

  for (int c0 = lo; c0 <= pos; c0 += 64) {
    const int key = c0 + lane;
    const bool valid = key <= pos;
    float s = -INFINITY;
    if (valid) {
      const int pg = bt[key / page];
      const long long off = (((long long)pg * Hkv + kvh) * page + key % page) * D;
      base[lane] = ((long long)pg * Hkv + kvh) * page * D + key % page;
      const typename P::V* kp = reinterpret_cast<const typename P::V*>(k_cache + off);
      float dot = 0.f;
      for (int d0 = 0; d0 < D; d0 += P::N) {
        float f[P::N];
        P::unpack(kp[d0 / P::N], f);
#pragma unroll
        for (int e = 0; e < P::N; ++e) dot = fmaf(qs[d0 + e], f[e], dot);
      }
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));      // finite: key c0 <= pos is valid
    const float alpha = expf(m - m_new);            // 0 on the first chunk (m = -inf)
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    ps[lane] = p;
    __syncthreads();
    const int nk = pos - c0 + 1 < 64 ? pos - c0 + 1 : 64;
#pragma unroll
    for (int i = 0; i < ATT_MAX_D / 64; ++i) acc[i] *= alpha;
    for (int j = 0; j < nk; ++j) {
      const float pj = ps[j];
      const T* vp = v_cache + base[j];
#pragma unroll
      for (int i = 0; i < ATT_MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) acc[i] = fmaf(pj, to_float(vp[(size_t)d * page]), acc[i]);
      }
    }
    __syncthreads();
    m = m_new;
  }
  const float inv = 1.0f / l;
  T* op = out + ((size_t)t * Hq + h) * D;
#pragma unroll
  for (int i = 0; i < ATT_MAX_D / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < D) op[d] = from_float<T>(acc[i] * inv);
  }
}

MIE_EXPORT const char* attention_last_error() { return g_mie_error; }

MIE_EXPORT int mie_paged_attention(const void* q, long q_stride, const void* k_cache, const void* v_cache, void* out,
                                   int dtype, const int* block_tables, int max_blocks, const int* token_row,
                                   const int* positions, int tokens, int Hq, int Hkv, int D, int page, float scale,
                                   int window, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (D % 16 || D < 16 || D > ATT_MAX_D) MIE_FAIL("paged_attention: head_dim %d (multiples of 16 up to %d)", D, ATT_MAX_D);
  if (Hkv <= 0 || Hq % Hkv) MIE_FAIL("paged_attention: %d query heads on %d kv heads", Hq, Hkv);
  if (Hq > 65535) MIE_FAIL("paged_attention: %d query heads is beyond the grid", Hq);
  if (page <= 0 || max_blocks <= 0) MIE_FAIL("paged_attention: page %d, max_blocks %d", page, max_blocks);
  if (q_stride < (long)Hq * D) MIE_FAIL("paged_attention: q row stride %ld < %d", q_stride, Hq * D);
  dim3 grid(tokens, Hq), block(64);
  if (dtype == MIE_F32)
    hipLaunchKernelGGL(paged_attention_kernel<float>, grid, block, 0, stream, (const float*)q, q_stride,
                       (const float*)k_cache, (const float*)v_cache, (float*)out, block_tables, max_blocks, token_row,
                       positions, Hq, Hkv, D, page, scale, window);
  else if (dtype == MIE_BF16)
    hipLaunchKernelGGL(paged_attention_kernel<bf16>, grid, block, 0, stream, (const bf16*)q, q_stride,
                       (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, block_tables, max_blocks, token_row,
                       positions, Hq, Hkv, D, page, scale, window);
  else
    MIE_FAIL("paged_attention: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("paged_attention");
  return 0;
}
