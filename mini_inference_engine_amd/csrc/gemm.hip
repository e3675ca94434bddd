// C = A W^T (+ bias): A [M, K], W [N, K] (the layout of a checkpoint's weight matrices),
// C [M, N], for any mix of float and bfloat16 operands, accumulated in true 32-bit FMAs.
//
// This is the kernel of the float32 path and the fallback for operand mixes the fast
// bfloat16 kernels do not take.  Every output element is one accumulator that adds its K
// products in increasing k, whatever M, N and the tile it falls in are: a token's result
// is bit-identical however the batch around it is cut.
// Also here: silu(gate) * up on the fused gate/up projection output.
#include "common.hpp"

#define GT 64      // tile of C
#define GK 16      // k per LDS stage
#define GPAD 4

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(const TA* __restrict__ A, long lda, const TW* __restrict__ W, long ldw, TC* __restrict__ C, long ldc,
               const float* __restrict__ bias, int M, int N, int K) {
  __shared__ float As[GK][GT + GPAD];
  __shared__ float Ws[GK][GT + GPAD];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      const int r = idx >> 4, c = idx & 15;
      const int k = k0 + c;
      float a = 0.f, w = 0.f;
      if (k < K) {
        if (m0 + r < M) a = to_float(A[(size_t)(m0 + r) * lda + k]);
        if (n0 + r < N) w = to_float(W[(size_t)(n0 + r) * ldw + k]);
      }
      As[c][r] = a;
      Ws[c][r] = w;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      C[(size_t)m * ldc + n] = from_float<TC>(v);
    }
  }
}

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, long ld_in, T* __restrict__ out, long ld_out, int rows, int inter) {
  const size_t total = (size_t)rows * inter;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t r = idx / inter, i = idx - r * inter;
    const float g = to_float(gu[r * ld_in + i]);
    const float u = to_float(gu[r * ld_in + inter + i]);
    out[r * ld_out + i] = from_float<T>(g / (1.0f + expf(-g)) * u);
  }
}

// bfloat16 rows whose gate and up halves start on 16 bytes: eight values a thread and a load
__global__ void __launch_bounds__(256)
silu_mul_bf16x8_kernel(const bf16* __restrict__ gu, long ld_in, bf16* __restrict__ out, long ld_out, int rows, int inter) {
  const int per_row = inter >> 3;
  const size_t total = (size_t)rows * per_row;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t r = idx / per_row, i = (idx - r * per_row) << 3;
    const uint4 g4 = *reinterpret_cast<const uint4*>(gu + r * ld_in + i);
    const uint4 u4 = *reinterpret_cast<const uint4*>(gu + r * ld_in + inter + i);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xFFFF0000u);
      const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xFFFF0000u);
      // g / (1 + e^-g) by the hardware's exp2 and reciprocal (each within an ulp or two of the exact value, far
      // below the bfloat16 rounding that follows): a tenth of the instructions of expf and a division
      const float s0 = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g0 * -1.4426950408889634f));
      const float s1 = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g1 * -1.4426950408889634f));
      const bf16 o0 = __float2bfloat16(g0 * s0 * u0), o1 = __float2bfloat16(g1 * s1 * u1);
      ow[j] = (uint32_t)__builtin_bit_cast(uint16_t, o0) | ((uint32_t)__builtin_bit_cast(uint16_t, o1) << 16);
    }
    *reinterpret_cast<uint4*>(out + r * ld_out + i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

MIE_EXPORT const char* gemm_last_error() { return g_mie_error; }

template <typename TA, typename TW>
static int launch_gemm_c(const void* A, long lda, const void* W, long ldw, void* C, int c_dtype, long ldc,
                         const float* bias, int M, int N, int K, hipStream_t s) {
  dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT), block(256);
  if (c_dtype == MIE_F32)
    hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, float>), grid, block, 0, s, (const TA*)A, lda, (const TW*)W, ldw,
                       (float*)C, ldc, bias, M, N, K);
  else if (c_dtype == MIE_BF16)
    hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, bf16>), grid, block, 0, s, (const TA*)A, lda, (const TW*)W, ldw,
                       (bf16*)C, ldc, bias, M, N, K);
  else
    MIE_FAIL("gemm: output dtype code %d", c_dtype);
  MIE_CHECK_LAUNCH("gemm");
  return 0;
}

MIE_EXPORT int mie_gemm_nt(const void* A, int a_dtype, long lda, const void* W, int w_dtype, long ldw, void* C,
                           int c_dtype, long ldc, const float* bias, int M, int N, int K, hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) MIE_FAIL("gemm: K = %d", K);
  if (lda < K || ldw < K || ldc < N) MIE_FAIL("gemm: leading dims %ld %ld %ld too small for K %d, N %d", lda, ldw, ldc, K, N);
  if ((M + GT - 1) / GT > 65535) MIE_FAIL("gemm: M = %d is beyond the grid", M);
  if (a_dtype == MIE_F32 && w_dtype == MIE_F32) return launch_gemm_c<float, float>(A, lda, W, ldw, C, c_dtype, ldc, bias, M, N, K, s);
  if (a_dtype == MIE_F32 && w_dtype == MIE_BF16) return launch_gemm_c<float, bf16>(A, lda, W, ldw, C, c_dtype, ldc, bias, M, N, K, s);
  if (a_dtype == MIE_BF16 && w_dtype == MIE_F32) return launch_gemm_c<bf16, float>(A, lda, W, ldw, C, c_dtype, ldc, bias, M, N, K, s);
  if (a_dtype == MIE_BF16 && w_dtype == MIE_BF16) return launch_gemm_c<bf16, bf16>(A, lda, W, ldw, C, c_dtype, ldc, bias, M, N, K, s);
  MIE_FAIL("gemm: dtype codes A %d, W %d", a_dtype, w_dtype);
}

MIE_EXPORT int mie_silu_mul(const void* gu, long ld_in, void* out, long ld_out, int dtype, int rows, int inter,
                            hipStream_t s) {
  if (rows <= 0 || inter <= 0) return 0;
  if (ld_in < 2L * inter || ld_out < inter) MIE_FAIL("silu_mul: leading dims %ld, %ld for intermediate %d", ld_in, ld_out, inter);
  const size_t total = (size_t)rows * inter;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 16384) blocks = 16384;
  if (dtype == MIE_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)gu, ld_in, (float*)out, ld_out, rows, inter);
  else if (dtype == MIE_BF16 && (inter & 7) == 0 && (ld_in & 7) == 0 && (ld_out & 7) == 0 &&
           (((uintptr_t)gu | (uintptr_t)out) & 15) == 0) {
    int b8 = (int)((total / 8 + 255) / 256);
    hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3(b8 > 16384 ? 16384 : b8), dim3(256), 0, s, (const bf16*)gu, ld_in,
                       (bf16*)out, ld_out, rows, inter);
  } else if (dtype == MIE_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16>, dim3(blocks), dim3(256), 0, s, (const bf16*)gu, ld_in, (bf16*)out, ld_out, rows, inter);
  else
    MIE_FAIL("silu_mul: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("silu_mul");
  return 0;
}
