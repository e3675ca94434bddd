// Next-token choice, one workgroup per row of 32-bit logits [R, V].
//
// temperature == 0:  argmax(logits), the lowest index among equal maxima.
// temperature  > 0:  argmax(logits / temperature + g_v), g_v = -log(-log(u_v)) Gumbel noise, which is a
//                    draw from softmax(logits / temperature).  u_v comes from a counter-based hash, not
//                    from generator state:
//   fmix(x): x ^= x >> 16; x *= 0x85EBCA6B; x ^= x >> 13; x *= 0xC2B2AE35; x ^= x >> 16   (32-bit)
//   key = fmix(fmix(fmix(seed_lo) ^ seed_hi) ^ counter)
//   x_v = fmix(key ^ fmix(v + 0x9E3779B9));   u_v = ((x_v >> 9) + 0.5) * 2^-23
// so the draw for (seed, counter) is the same in any batch.  Greedy and sampled rows share the
// kernel; nothing is decided on the host.
#include "common.hpp"

__device__ __forceinline__ uint32_t fmix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x85EBCA6Bu;
  x ^= x >> 13;
  x *= 0xC2B2AE35u;
  x ^= x >> 16;
  return x;
}

#define SAMPLE_THREADS 1024

// One candidate: its value after temperature and noise, kept if it beats the best so far.
__device__ __forceinline__ void sample_consider(float z, int v, bool noisy, float inv_t, uint32_t key, float& bv, int& bi) {
  if (noisy) {
    const uint32_t x = fmix32(key ^ fmix32((uint32_t)v + 0x9E3779B9u));
    const float u = ((float)(x >> 9) + 0.5f) * 1.1920928955078125e-07f;   // 2^-23
    z = z * inv_t - logf(-logf(u));
  }
  if (z > bv || (z == bv && v < bi)) { bv = z; bi = v; }
}

// VEC: the row is read four values at a time (needs a 16-byte aligned row), several reads in flight a thread.
template <bool VEC>
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, long ld, const float* __restrict__ temperatures,
              const long long* __restrict__ seeds, const int* __restrict__ counters, int* __restrict__ out, int V) {
  __shared__ float best_v[SAMPLE_THREADS / 64];
  __shared__ int best_i[SAMPLE_THREADS / 64];
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * ld;
  const float temp = temperatures[r];
  const bool noisy = temp > 0.f;
  const float inv_t = noisy ? 1.0f / temp : 1.0f;
  uint32_t key = 0;
  if (noisy) {
    const unsigned long long seed = (unsigned long long)seeds[r];
    key = fmix32(fmix32(fmix32((uint32_t)seed) ^ (uint32_t)(seed >> 32)) ^ (uint32_t)counters[r]);
  }
  float bv = -INFINITY;
  int bi = 0x7FFFFFFF;
  if (VEC) {
    const int V4 = V & ~3;
#pragma unroll 4
    for (int v = threadIdx.x * 4; v < V4; v += SAMPLE_THREADS * 4) {
      const float4 z = *reinterpret_cast<const float4*>(row + v);
      sample_consider(z.x, v, noisy, inv_t, key, bv, bi);
      sample_consider(z.y, v + 1, noisy, inv_t, key, bv, bi);
      sample_consider(z.z, v + 2, noisy, inv_t, key, bv, bi);
      sample_consider(z.w, v + 3, noisy, inv_t, key, bv, bi);
    }
    if (V4 + (int)threadIdx.x < V) sample_consider(row[V4 + threadIdx.x], V4 + threadIdx.x, noisy, inv_t, key, bv, bi);
  } else {
#pragma unroll 4
    for (int v = threadIdx.x; v < V; v += SAMPLE_THREADS) sample_consider(row[v], v, noisy, inv_t, key, bv, bi);
  }
  // NaN logits never win a comparison; a row of only NaN yields index 0 below.
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) { best_v[w] = bv; best_i[w] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < SAMPLE_THREADS / 64; ++i)
      if (best_v[i] > bv || (best_v[i] == bv && best_i[i] < bi)) { bv = best_v[i]; bi = best_i[i]; }
    out[r] = bi == 0x7FFFFFFF ? 0 : bi;
  }
}

MIE_EXPORT const char* sampling_last_error() { return g_mie_error; }

MIE_EXPORT int mie_sample(const float* logits, long ld, const float* temperatures, const long long* seeds,
                          const int* counters, int* out, int rows, int V, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (V <= 0 || ld < V) MIE_FAIL("sample: vocabulary %d, leading dim %ld", V, ld);
  if (((uintptr_t)logits & 15) == 0 && (ld & 3) == 0)
    hipLaunchKernelGGL(sample_kernel<true>, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, ld, temperatures, seeds,
                       counters, out, V);
  else
    hipLaunchKernelGGL(sample_kernel<false>, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, ld, temperatures,
                       seeds, counters, out, V);
  MIE_CHECK_LAUNCH("sample");
  return 0;
}
