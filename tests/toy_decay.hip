// A test fixture, not part of the engine: the kernel of the toy mixer of tests/test_generality.py, built and
// loaded through the engine's kernel-module registry from outside the package.
//   s_t = decay * s_{t-1} + x_t  per request;  out_t = s_t;  the state lives in the request's slot.
// One workgroup a row (a request's tokens of this step), one thread a column.
#include "common.hpp"

__global__ void __launch_bounds__(256)
toy_decay_kernel(const float* __restrict__ x, float* __restrict__ out, float* __restrict__ state,
                 const int* __restrict__ row_start, const int* __restrict__ slots, float decay, int width) {
  const int r = blockIdx.x;
  const int a = row_start[r], b = row_start[r + 1];
  float* s_row = state + (size_t)slots[r] * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float s = s_row[c];
    for (int t = a; t < b; ++t) {
      s = decay * s + x[(size_t)t * width + c];
      out[(size_t)t * width + c] = s;
    }
    s_row[c] = s;
  }
}

MIE_EXPORT const char* toy_decay_last_error() { return g_mie_error; }

// x, out [tokens, width] float32; state [slots, width] float32; row_start [rows + 1], slots [rows] int32
MIE_EXPORT int toy_decay_scan(const float* x, float* out, float* state, const int* row_start, const int* slots,
                              int rows, int width, float decay, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (width <= 0 || !x || !out || !state || !row_start || !slots) MIE_FAIL("toy_decay_scan: operands");
  hipLaunchKernelGGL(toy_decay_kernel, dim3(rows), dim3(256), 0, stream, x, out, state, row_start, slots, decay, width);
  MIE_CHECK_LAUNCH("toy_decay_scan");
  return 0;
}
