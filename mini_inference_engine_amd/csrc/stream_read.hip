// A measurement, not a part of any model: how fast this GPU streams memory that is only read, which is what a
// decode step does with its weights and its cache.  Every thread reads 16 bytes at a time, four reads in flight,
// the workgroups interleaved over the buffer; the words read are folded into one value a thread and stored, so
// that the reads cannot be dropped (the stores are 1/1024 of the bytes for a buffer of 1 GiB).
#include "common.hpp"

#define STREAM_THREADS 256

template <bool NONTEMPORAL>
__global__ void __launch_bounds__(STREAM_THREADS)
stream_read_kernel(const uint4* __restrict__ src, long n16, uint32_t* __restrict__ out) {
  const long stride = (long)gridDim.x * STREAM_THREADS;
  long i = (long)blockIdx.x * STREAM_THREADS + threadIdx.x;
  uint32_t acc = 0;
  auto read = [&](long at) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(src + at);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = NONTEMPORAL ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p))
                                : *reinterpret_cast<const u32x4*>(p);
    return v.x ^ v.y ^ v.z ^ v.w;
  };
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint32_t a = read(i), b = read(i + stride), c = read(i + 2 * stride), d = read(i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n16; i += stride) acc ^= read(i);
  out[(long)blockIdx.x * STREAM_THREADS + threadIdx.x] = acc;
}

MIE_EXPORT const char* stream_read_last_error() { return g_mie_error; }

// ``out`` holds 256 words for each of the ``workgroups`` (1 to 65536) the launch uses.
MIE_EXPORT int mie_stream_read(const void* src, long bytes, uint32_t* out, int workgroups, int nontemporal, hipStream_t stream) {
  if (bytes <= 0 || (bytes & 15) || ((uintptr_t)src & 15)) MIE_FAIL("stream_read: %ld bytes at %p: multiples of 16 wanted", bytes, src);
  if (workgroups < 1 || workgroups > 65536) MIE_FAIL("stream_read: %d workgroups", workgroups);
  const int grid = workgroups;
  if (nontemporal)
    hipLaunchKernelGGL(stream_read_kernel<true>, dim3(grid), dim3(STREAM_THREADS), 0, stream, (const uint4*)src, bytes / 16, out);
  else
    hipLaunchKernelGGL(stream_read_kernel<false>, dim3(grid), dim3(STREAM_THREADS), 0, stream, (const uint4*)src, bytes / 16, out);
  MIE_CHECK_LAUNCH("stream_read");
  return 0;
}
