// Token embedding into the 32-bit residual stream, and the residual add fused with RMSNorm.
//
// embedding:    stream[t, :] = float(table[ids[t], :])
// add_rmsnorm:  r = stream[row] (+ float(x[row]));  stream[row] = r (unless rows are gathered);
//               y[row] = r * (1 / sqrt(mean(r^2) + eps)) * weight, rounded once to y's type.
// One workgroup per row; the row's sum of squares is reduced in an order that depends only on
// the row width, so a token's result does not depend on what else is in the batch.
#include "common.hpp"

template <typename TT>
__global__ void embedding_kernel(const int* __restrict__ ids, const TT* __restrict__ table, float* __restrict__ out,
                                 int width, int vocab, const int* __restrict__ taken_from,
                                 const int* __restrict__ earlier_tokens) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (taken_from) {            // a token the host does not know yet: entry taken_from[t] of the tokens chosen last
    const int j = taken_from[t];
    if (j >= 0) id = earlier_tokens[j];
  }
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // ids are validated on the host; never read outside
  const TT* src = table + (size_t)id * width;
  float* dst = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_float(src[i]);
}

#define NORM_THREADS 256
#define NORM_CACHE 16

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(NORM_THREADS)
add_rmsnorm_kernel(const TX* __restrict__ x, float* __restrict__ stream, const TW* __restrict__ weight,
                   TY* __restrict__ y, const int* __restrict__ rows, int width, float eps) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int row = rows ? rows[out_row] : out_row;
  float* sr = stream + (size_t)row * width;
  const TX* xr = x ? x + (size_t)row * width : nullptr;
  float cache[NORM_CACHE];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NORM_CACHE; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    float r = 0.f;
    if (i < width) {
      r = sr[i];
      if (xr) r += to_float(xr[i]);
      if (xr && !rows) sr[i] = r;
    }
    cache[k] = r;
    ss += r * r;
  }
  for (int i = threadIdx.x + NORM_CACHE * NORM_THREADS; i < width; i += NORM_THREADS) {
    float r = sr[i];
    if (xr) r += to_float(xr[i]);
    if (xr && !rows) sr[i] = r;
    ss += r * r;
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)width + eps);
  TY* yr = y + (size_t)out_row * width;
#pragma unroll
  for (int k = 0; k < NORM_CACHE; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    if (i < width) yr[i] = from_float<TY>(cache[k] * rstd * to_float(weight[i]));
  }
  for (int i = threadIdx.x + NORM_CACHE * NORM_THREADS; i < width; i += NORM_THREADS) {
    float r = sr[i];
    if (xr && rows) r += to_float(xr[i]);   // gathered rows were not written back
    yr[i] = from_float<TY>(r * rstd * to_float(weight[i]));
  }
}


// Few rows (a decode step): the whole cost is latency, so every load of a row (stream, pending x and
// weight) is issued before anything is reduced, 4 elements a lane at a time.  Same arithmetic and the
// same order of the block reduction inputs as above is not required: the fast path is taken for a row
// whenever width % 4 == 0 and width <= 4 * NORM_FAST_THREADS * NORM_FAST_VEC, whatever the batch is,
// so a row's result still does not depend on the batch.
#define NORM_FAST_THREADS 256
#define NORM_FAST_VEC 8      // float4 groups per thread: widths up to 8192

// four elements as they lie in memory, and as numbers
template <typename T> struct Raw4;
template <> struct Raw4<float> { float4 v; };
template <> struct Raw4<bf16> { uint2 v; };
__device__ __forceinline__ Raw4<float> load_raw(const float* p) { return Raw4<float>{*reinterpret_cast<const float4*>(p)}; }
__device__ __forceinline__ Raw4<bf16> load_raw(const bf16* p) { return Raw4<bf16>{*reinterpret_cast<const uint2*>(p)}; }
__device__ __forceinline__ float4 to_float4(const Raw4<float>& r) { return r.v; }
__device__ __forceinline__ float4 to_float4(const Raw4<bf16>& r) {
  return make_float4(__uint_as_float(r.v.x << 16), __uint_as_float(r.v.x & 0xFFFF0000u), __uint_as_float(r.v.y << 16),
                     __uint_as_float(r.v.y & 0xFFFF0000u));
}
template <typename T> __device__ __forceinline__ float4 load4(const T* p);
template <> __device__ __forceinline__ float4 load4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 load4<bf16>(const bf16* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xFFFF0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xFFFF0000u));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.x)) | ((uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.y)) << 16);
  u.y = (uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.z)) | ((uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// VEC: float4 groups a thread holds (the width is at most 4 * NORM_FAST_THREADS * VEC): as few as the width
// needs, so that narrow rows do not pay in registers, and so in resident workgroups, for wide ones
template <typename TX, typename TW, typename TY, int VEC>
__global__ void __launch_bounds__(NORM_FAST_THREADS)
add_rmsnorm_fast_kernel(const TX* __restrict__ x, float* __restrict__ stream, const TW* __restrict__ weight,
                        TY* __restrict__ y, const int* __restrict__ rows, int width, float eps) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int row = rows ? rows[out_row] : out_row;
  float* sr = stream + (size_t)row * width;
  const TX* xr = x ? x + (size_t)row * width : nullptr;
  // first every load, as it comes from memory (a conversion or an add where a value is loaded would make
  // the compiler wait for it there, one memory latency per group of four instead of one in all)
  Raw4<float> r_raw[VEC];
  Raw4<TW> w_raw[VEC];
  Raw4<TX> a_raw[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int i = (threadIdx.x + k * NORM_FAST_THREADS) * 4;
    r_raw[k] = Raw4<float>{};
    w_raw[k] = Raw4<TW>{};
    a_raw[k] = Raw4<TX>{};
    if (i < width) {
      r_raw[k] = load_raw(sr + i);
      w_raw[k] = load_raw(weight + i);
      if (xr) a_raw[k] = load_raw(xr + i);
    }
  }
  float4 r[VEC], w[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    r[k] = to_float4(r_raw[k]);
    w[k] = to_float4(w_raw[k]);
    const float4 a = to_float4(a_raw[k]);          // zeros where nothing was loaded
    r[k].x += a.x; r[k].y += a.y; r[k].z += a.z; r[k].w += a.w;
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    ss = fmaf(r[k].x, r[k].x, ss); ss = fmaf(r[k].y, r[k].y, ss);
    ss = fmaf(r[k].z, r[k].z, ss); ss = fmaf(r[k].w, r[k].w, ss);
    const int i = (threadIdx.x + k * NORM_FAST_THREADS) * 4;
    if (xr && !rows && i < width) store4(sr + i, r[k]);
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)width + eps);
  TY* yr = y + (size_t)out_row * width;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int i = (threadIdx.x + k * NORM_FAST_THREADS) * 4;
    if (i < width)
      store4(yr + i, make_float4(r[k].x * rstd * w[k].x, r[k].y * rstd * w[k].y, r[k].z * rstd * w[k].z,
                                 r[k].w * rstd * w[k].w));
  }
}

MIE_EXPORT const char* embed_norm_last_error() { return g_mie_error; }

// taken_from (or null) [tokens]: where >= 0, the token is earlier_tokens[taken_from[t]] instead of ids[t]
// (a token chosen by the step before, which the host has not seen yet).
MIE_EXPORT int mie_embedding(const int* ids, const void* table, int table_dtype, float* out, int tokens, int width,
                             int vocab, const int* taken_from, const int* earlier_tokens, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width <= 0 || vocab <= 0) MIE_FAIL("embedding: width %d, vocab %d", width, vocab);
  if (taken_from && !earlier_tokens) MIE_FAIL("embedding: taken_from without the tokens to take from");
  dim3 grid(tokens), block(256);
  if (table_dtype == MIE_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, grid, block, 0, stream, ids, (const float*)table, out, width, vocab,
                       taken_from, earlier_tokens);
  else if (table_dtype == MIE_BF16)
    hipLaunchKernelGGL(embedding_kernel<bf16>, grid, block, 0, stream, ids, (const bf16*)table, out, width, vocab,
                       taken_from, earlier_tokens);
  else
    MIE_FAIL("embedding: table dtype code %d", table_dtype);
  MIE_CHECK_LAUNCH("embedding");
  return 0;
}

template <typename TX, typename TW>
static int launch_norm(const void* x, float* stream, const void* w, void* y, int y_dtype, const int* rows, int n_rows,
                       int width, float eps, hipStream_t s) {
  dim3 grid(n_rows), block(NORM_THREADS);
  // the vector kernel whenever the width allows it (a property of the model, not of the batch)
  const bool fast = width % 4 == 0 && width <= 4 * NORM_FAST_THREADS * NORM_FAST_VEC &&
                    (((uintptr_t)x | (uintptr_t)stream | (uintptr_t)w | (uintptr_t)y) & 15) == 0;
  if (y_dtype != MIE_F32 && y_dtype != MIE_BF16) MIE_FAIL("add_rmsnorm: output dtype code %d", y_dtype);
  if (fast) {
#define NORM_FAST_LAUNCH(TY_, V_)                                                                                     \
  hipLaunchKernelGGL((add_rmsnorm_fast_kernel<TX, TW, TY_, V_>), grid, dim3(NORM_FAST_THREADS), 0, s, (const TX*)x, \
                     stream, (const TW*)w, (TY_*)y, rows, width, eps)
    const int groups = (width / 4 + NORM_FAST_THREADS - 1) / NORM_FAST_THREADS;
    if (y_dtype == MIE_F32) {
      if (groups <= 2) NORM_FAST_LAUNCH(float, 2);
      else if (groups <= 4) NORM_FAST_LAUNCH(float, 4);
      else NORM_FAST_LAUNCH(float, NORM_FAST_VEC);
    } else {
      if (groups <= 2) NORM_FAST_LAUNCH(bf16, 2);
      else if (groups <= 4) NORM_FAST_LAUNCH(bf16, 4);
      else NORM_FAST_LAUNCH(bf16, NORM_FAST_VEC);
    }
#undef NORM_FAST_LAUNCH
  }
  else if (y_dtype == MIE_F32)
    hipLaunchKernelGGL((add_rmsnorm_kernel<TX, TW, float>), grid, block, 0, s, (const TX*)x, stream, (const TW*)w,
                       (float*)y, rows, width, eps);
  else
    hipLaunchKernelGGL((add_rmsnorm_kernel<TX, TW, bf16>), grid, block, 0, s, (const TX*)x, stream, (const TW*)w,
                       (bf16*)y, rows, width, eps);
  MIE_CHECK_LAUNCH("add_rmsnorm");
  return 0;
}

// x may be null (nothing to add).  rows may be null (all n_rows rows, stream updated in place).
MIE_EXPORT int mie_add_rmsnorm(const void* x, int x_dtype, float* stream, const void* weight, int w_dtype, void* y,
                               int y_dtype, const int* rows, int n_rows, int width, float eps, hipStream_t s) {
  if (n_rows <= 0) return 0;
  if (width <= 0) MIE_FAIL("add_rmsnorm: width %d", width);
  if (x_dtype == MIE_F32 && w_dtype == MIE_F32) return launch_norm<float, float>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  if (x_dtype == MIE_F32 && w_dtype == MIE_BF16) return launch_norm<float, bf16>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  if (x_dtype == MIE_BF16 && w_dtype == MIE_F32) return launch_norm<bf16, float>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  if (x_dtype == MIE_BF16 && w_dtype == MIE_BF16) return launch_norm<bf16, bf16>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  MIE_FAIL("add_rmsnorm: dtype codes x %d, weight %d", x_dtype, w_dtype);
}
