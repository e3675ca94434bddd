// Matrix products of the bfloat16 path with 17 to 128 rows and a narrow weight (N up to a few thousand):
// decode steps of many requests.  The few-row kernel (gemm_bf16.hip) gives every 16 weight rows a
// workgroup that reads all of x, which at 64 rows is four times the weights' bytes; a library product
// runs such a shape on a few dozen workgroups.  Here
//
//   part[s, m, n] = sum over the k of split s of x[m, k] W[n, k]
//
// a workgroup of 4 waves owns 64 weight rows and one contiguous range of K (the split); k-steps of W
// and of x (all rows) are brought into a ring of LDS stages by loads that write the LDS directly, 1 KB a
// fragment (16 rows x 32 k), so x is read once per 64 weight rows; wave w multiplies its 16 weight rows
// with v_mfma_f32_16x16x32_bf16.  The split's sums go out as float32 partial results.
// A fragment is brought in by lane 4 r + b reading k-block b ^ (r / 4) % 4 of row r (16 bytes): a quarter
// wave then reads 64 contiguous bytes of 4 rows (in the matrix instruction's own order, lane 16 b + r, it
// touches 16 cache lines for 16 bytes each, and the address unit's line look-ups bound the kernel), and the
// permutation of the blocks spreads the fragment reads (lane 16 b + r reads slot 4 r + (b ^ (r / 4) % 4))
// over all banks.
// The number of splits is chosen by the caller from the weight's shape alone, so a row's result does
// not depend on the batch it is in.
//
// The kernels that follow add the partial results up in split order and do what comes after the product:
//   reduce_rows:     store (bfloat16 / float32), or add into the 32-bit stream, or add and RMSNorm for
//                    the norm that reads the stream next (one workgroup a row, as the norm kernel);
//   reduce_rope_kv:  the q/k/v projection: rotary on q and k, q out, k and v into their cache slots.
#include "common.hpp"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

union Frag {
  bf16x8 v;
  uint4 q;
};

constexpr int MID_WAVES = 4;      // waves a workgroup = 16-row weight tiles a workgroup
constexpr int MID_KC = 2;         // k-steps (of 32) a stage
constexpr int MID_STAGES = 4;     // stages in the ring (eight were measured: no faster)
constexpr int FRAG_BYTES = 1024;  // one operand fragment: 64 lanes x 16 bytes

// wait until at most n vector memory loads of this wave are still on their way
#define MID_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// The fragments of one k-step out of the LDS: the wave's weight fragment (at wbase) and the x fragments of all
// row tiles (1 KB apart from xbase), read and waited for in one piece of assembly.  The compiler knows nothing
// of the loads that write the LDS, so a read of the LDS it could see would make it wait for every load on its
// way; and it must never see a register whose value is still to arrive (it may move it), so the wait is part
// of the same piece.  OFF: byte offset of the k-step within the stage, XOFF: of its first x fragment.
template <int MT, int OFF, int XOFF>
struct LdsFragments;
template <int OFF, int XOFF>
struct LdsFragments<4, OFF, XOFF> {
  static __device__ __forceinline__ void read(uint32_t wbase, uint32_t xbase, u32x4& w, u32x4 (&x)[4]) {
    asm volatile(
      "ds_read_b128 %0, %5 offset:%7\n\t"
      "ds_read_b128 %1, %6 offset:%8\n\t"
      "ds_read_b128 %2, %6 offset:%8+1024\n\t"
      "ds_read_b128 %3, %6 offset:%8+2048\n\t"
      "ds_read_b128 %4, %6 offset:%8+3072\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(w), "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3])
      : "v"(wbase), "v"(xbase), "n"(OFF), "n"(XOFF)
      : "memory");
  }
};
template <int OFF, int XOFF>
struct LdsFragments<8, OFF, XOFF> {
  static __device__ __forceinline__ void read(uint32_t wbase, uint32_t xbase, u32x4& w, u32x4 (&x)[8]) {
    asm volatile(
      "ds_read_b128 %0, %9 offset:%11\n\t"
      "ds_read_b128 %1, %10 offset:%12\n\t"
      "ds_read_b128 %2, %10 offset:%12+1024\n\t"
      "ds_read_b128 %3, %10 offset:%12+2048\n\t"
      "ds_read_b128 %4, %10 offset:%12+3072\n\t"
      "ds_read_b128 %5, %10 offset:%12+4096\n\t"
      "ds_read_b128 %6, %10 offset:%12+5120\n\t"
      "ds_read_b128 %7, %10 offset:%12+6144\n\t"
      "ds_read_b128 %8, %10 offset:%12+7168\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(w), "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6]), "=&v"(x[7])
      : "v"(wbase), "v"(xbase), "n"(OFF), "n"(XOFF)
      : "memory");
  }
};

// One stage = KC k-steps; a k-step holds the waves' weight fragments, then the x fragments of the row tiles.
template <int MT, int kc>
struct StageReader {
  static constexpr int SF = MID_WAVES + MT;
  static_assert(FRAG_BYTES == 1024, "the offsets in LdsFragments");
  static __device__ __forceinline__ void run(uint32_t base, uint32_t wbase, f32x4 (&acc)[MT]) {
    u32x4 w, x[MT];
    LdsFragments<MT, kc * SF * FRAG_BYTES, (kc * SF + MID_WAVES) * FRAG_BYTES>::read(wbase, base, w, x);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      Frag a, b;
      a.q = *reinterpret_cast<uint4*>(&x[mt]);
      b.q = *reinterpret_cast<uint4*>(&w);
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[mt], 0, 0, 0);
    }
    if constexpr (kc + 1 < MID_KC) StageReader<MT, kc + 1>::run(base, wbase, acc);
  }
};

// grid (ceil(N / 64), splits).  zeros: 64 bytes of zeros in device memory (what a k-step beyond the range
// or beyond K loads instead, so that every load is unconditional).  part [splits, M, N] float32.
template <int MT>
__global__ void __launch_bounds__(MID_WAVES * 64)
mid_gemm_kernel(const bf16* __restrict__ X, long ldx, const bf16* __restrict__ W, long ldw, float* __restrict__ part,
                int M, int N, int K, int kper, const bf16* __restrict__ zeros) {
  extern __shared__ __align__(16) char lds[];
  constexpr int SF = MID_WAVES + MT;                       // fragments a k-step
  constexpr int STAGE_BYTES = MID_KC * SF * FRAG_BYTES;
  static_assert((MT * MID_KC) % MID_WAVES == 0, "the x fragments of a stage must divide over the waves");
  constexpr int XL = MT * MID_KC / MID_WAVES;              // x fragments a wave brings in per stage
  constexpr int L = MID_KC + XL;                           // loads a wave issues per stage
  static_assert((MID_STAGES - 2) * L <= 63, "more loads in flight than the counter holds");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int lrow = lane >> 2, lkb = (lane & 3) ^ ((lrow >> 2) & 3);     // the row and k-block this lane brings in
  const int rslot = col * 4 + (kb ^ ((col >> 2) & 3));                  // where this lane's piece of a fragment sits
  const int ksteps = (K + 31) >> 5;
  const int ksA = blockIdx.y * kper, ksB = ksA + kper < ksteps ? ksA + kper : ksteps;
  const int nst = (ksB - ksA + MID_KC - 1) / MID_KC;
  const int n = (blockIdx.x * MID_WAVES + wave) * 16 + col;
  const int nl = (blockIdx.x * MID_WAVES + wave) * 16 + lrow;
  const bf16* wrow = W + (size_t)(nl < N ? nl : N - 1) * ldw + lkb * 8;
  const bf16* xptr[XL];
  int xkc[XL], xlds[XL];
#pragma unroll
  for (int j = 0; j < XL; ++j) {
    const int f = wave * XL + j, kc = f / MT, mt = f % MT;
    const int m = mt * 16 + lrow;
    xptr[j] = X + (size_t)(m < M ? m : 0) * ldx + kc * 32 + lkb * 8;
    xkc[j] = kc;
    xlds[j] = (kc * SF + MID_WAVES + mt) * FRAG_BYTES;
  }
  const bf16* zero_lane = zeros + lkb * 8;     // a per-lane address, so that choosing it is a select and no branch
  auto issue = [&](int s) {
    char* base = lds + (s % MID_STAGES) * STAGE_BYTES;
    const int ks = ksA + s * MID_KC;
#pragma unroll
    for (int kc = 0; kc < MID_KC; ++kc) {
      const bool ok = ks + kc < ksB && (ks + kc) * 32 + lkb * 8 < K;
      const bf16* src = ok ? wrow + (size_t)(ks + kc) * 32 : zero_lane;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(base + (kc * SF + wave) * FRAG_BYTES), 16, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < XL; ++j) {
      const bool ok = ks + xkc[j] < ksB && (ks + xkc[j]) * 32 + lkb * 8 < K;
      const bf16* src = ok ? xptr[j] + (size_t)ks * 32 : zero_lane;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(base + xlds[j]), 16, 0, 0);
    }
  };
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
  // stages beyond the split's range load zeros only, so the ring is always filled and drained the same way
  for (int s = 0; s < MID_STAGES - 1; ++s) issue(s);
  for (int it = 0; it < nst; ++it) {
    MID_VMCNT((MID_STAGES - 2) * L);           // this wave's loads of stage `it` have landed
    __builtin_amdgcn_s_barrier();              // and everybody else's; everybody is done reading stage it - 1
    issue(it + MID_STAGES - 1);                // into the buffer stage it - 1 used
    const uint32_t base = lds0 + (it % MID_STAGES) * STAGE_BYTES + rslot * 16;
    StageReader<MT, 0>::run(base, base + wave * FRAG_BYTES, acc);
  }
  MID_VMCNT(0);                                // nothing of this wave may still be writing the LDS when it ends
  float* out = part + (size_t)blockIdx.y * M * N;
  // acc[mt][i]: x row mt * 16 + 4 kb + i (the A operand's rows), weight row n (the B operand's column)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = mt * 16 + kb * 4 + i;
      if (m < M && n < N) out[(size_t)m * N + n] = acc[mt][i];
    }
}

// ---------------------------------------------------------------------------- after the product
enum { RED_STORE_BF16 = 0, RED_STORE_F32 = 1, RED_ADD = 2, RED_ADD_NORM = 3 };
constexpr int RED_THREADS = 512;
constexpr int RED_VEC = 4;        // float4 a thread: rows up to 8192 wide

__device__ __forceinline__ void store_bf16x4(bf16* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.x)) | ((uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.y)) << 16);
  u.y = (uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.z)) | ((uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// One workgroup a row; N a multiple of 4, at most 4 * RED_THREADS * RED_VEC.  y = sum of the splits in
// split order.  STORE: out[m, :] = y.  ADD: stream[m, :] += y.  ADD_NORM: also x_next[m, :] =
// bf16(stream * rsqrt(mean(stream^2) + eps) * g), the RMSNorm that reads the stream next.
template <int MODE>
__global__ void __launch_bounds__(RED_THREADS)
reduce_rows_kernel(const float* __restrict__ part, int splits, size_t split_stride, int N, void* __restrict__ out,
                   long ldo, float* __restrict__ stream, const void* __restrict__ g, int g_f32,
                   bf16* __restrict__ x_next, long ldx_next, float eps) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const float* pr = part + (size_t)m * N;
  f32x4 y[RED_VEC];
  float4 w[RED_VEC];
#pragma unroll
  for (int k = 0; k < RED_VEC; ++k) {
    const int i = (threadIdx.x + k * RED_THREADS) * 4;
    y[k] = f32x4{0.f, 0.f, 0.f, 0.f};
    w[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < N) {
      if (MODE == RED_ADD || MODE == RED_ADD_NORM) y[k] = *reinterpret_cast<const f32x4*>(stream + (size_t)m * N + i);
      if (MODE == RED_ADD_NORM) {
        if (g_f32) {
          w[k] = *reinterpret_cast<const float4*>((const float*)g + i);
        } else {
          const uint2 u = *reinterpret_cast<const uint2*>((const uint16_t*)g + i);
          w[k] = make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xFFFF0000u), __uint_as_float(u.y << 16),
                             __uint_as_float(u.y & 0xFFFF0000u));
        }
      }
      add_splits(y[k], reinterpret_cast<const f32x4*>(pr + i), splits, split_stride / 4);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < RED_VEC; ++k) {
    const int i = (threadIdx.x + k * RED_THREADS) * 4;
    if (i >= N) continue;
    const float4 v = make_float4(y[k][0], y[k][1], y[k][2], y[k][3]);
    if (MODE == RED_STORE_BF16) store_bf16x4((bf16*)out + (size_t)m * ldo + i, v);
    if (MODE == RED_STORE_F32) *reinterpret_cast<float4*>((float*)out + (size_t)m * ldo + i) = v;
    if (MODE == RED_ADD || MODE == RED_ADD_NORM) *reinterpret_cast<float4*>(stream + (size_t)m * N + i) = v;
    ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss);
    ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss);
  }
  if (MODE != RED_ADD_NORM) return;
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)N + eps);
#pragma unroll
  for (int k = 0; k < RED_VEC; ++k) {
    const int i = (threadIdx.x + k * RED_THREADS) * 4;
    if (i >= N) continue;
    store_bf16x4(x_next + (size_t)m * ldx_next + i,
                 make_float4(y[k][0] * rstd * w[k].x, y[k][1] * rstd * w[k].y, y[k][2] * rstd * w[k].z, y[k][3] * rstd * w[k].w));
  }
}

// The q/k/v projection's partial results, grid (rows, ceil(heads / 4)), a wave a head (q heads, then k heads,
// then v heads): rotary (half-split pairs over the whole head, 32-bit angles) on the q and k heads,
// q [M, Hq D] out, k and v into cache slot slots[m] (k_cache [pages, Hkv, page, D], v_cache [pages, Hkv, D, page]).
__global__ void __launch_bounds__(256)
reduce_rope_kv_kernel(const float* __restrict__ part, int splits, size_t split_stride, bf16* __restrict__ q_out, long ldq,
                      const int* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                      const int* __restrict__ slots, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache, int Hq,
                      int Hkv, int D, int page) {
  const int m = blockIdx.x;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (head >= Hq + 2 * Hkv) return;
  const int N = (Hq + 2 * Hkv) * D;
  const float* pr = part + (size_t)m * N + (size_t)head * D;
  const int half = D >> 1;
  const int pos = positions[m], slot = slots[m];
  if (head < Hq + Hkv) {
    const float* cr = cos_t + (size_t)pos * half;
    const float* sr = sin_t + (size_t)pos * half;
    bf16* dst = head < Hq ? q_out + (size_t)m * ldq + (size_t)head * D
                          : k_cache + (((size_t)(slot / page) * Hkv + (head - Hq)) * page + (size_t)(slot % page)) * D;
    for (int j = lane; j < half; j += 64) {
      const float c = cr[j], sn = sr[j];
      float x1 = 0.f, x2 = 0.f;
      add_splits(x1, pr + j, splits, split_stride);
      add_splits(x2, pr + j + half, splits, split_stride);
      float o1, o2;
      rotate_pair(x1, x2, c, sn, o1, o2);
      dst[j] = __float2bfloat16(o1);
      dst[j + half] = __float2bfloat16(o2);
    }
  } else {
    bf16* dst = v_cache + ((size_t)(slot / page) * Hkv + (head - Hq - Hkv)) * page * D + (size_t)(slot % page);
    for (int d = lane; d < D; d += 64) {
      float v = 0.f;
      add_splits(v, pr + d, splits, split_stride);
      dst[(size_t)d * page] = __float2bfloat16(v);
    }
  }
}

MIE_EXPORT const char* gemm_mid_bf16_last_error() { return g_mie_error; }
MIE_EXPORT int mie_mid_max_rows() { return 128; }

// How the caller has to cut K: k-steps a split for ``splits`` wanted splits, and the number of splits that gives.
static void cut_k(int K, int wanted, int* kper, int* splits) {
  const int ksteps = (K + 31) / 32;
  int per = (ksteps + wanted - 1) / wanted;
  per = (per + MID_KC - 1) / MID_KC * MID_KC;
  *kper = per;
  *splits = (ksteps + per - 1) / per;
}

// The number of splits mie_mid_gemm will really make of ``wanted`` (the caller sizes ``part`` by it).
MIE_EXPORT int mie_mid_splits(int K, int wanted) {
  if (K <= 0 || wanted <= 0) return 0;
  int kper, splits;
  cut_k(K, wanted, &kper, &splits);
  return splits;
}

template <int MT>
static int launch_mid(dim3 grid, hipStream_t s, const bf16* X, long ldx, const bf16* W, long ldw, float* part, int M, int N,
                      int K, int kper, const bf16* zeros) {
  constexpr int lds_bytes = MID_STAGES * MID_KC * (MID_WAVES + MT) * FRAG_BYTES;
  if (lds_bytes > 64 * 1024) {
    // more LDS than a kernel gets by default: asked for once per device
    static bool raised[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) MIE_FAIL("mid_gemm: no current device");
    if (!raised[dev]) {
      hipError_t e = hipFuncSetAttribute((const void*)mid_gemm_kernel<MT>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) MIE_FAIL("mid_gemm: %d bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
      raised[dev] = true;
    }
  }
  hipLaunchKernelGGL((mid_gemm_kernel<MT>), grid, dim3(MID_WAVES * 64), lds_bytes, s, X, ldx, W, ldw, part, M, N, K, kper, zeros);
  MIE_CHECK_LAUNCH("mid_gemm");
  return 0;
}

// X [M, K], W [N, K] bfloat16 (16-byte aligned, leading dims multiples of 8, K a multiple of 8), M <= 128.
// part [mie_mid_splits(K, wanted_splits), M, N] float32.  zeros: 64 zero bytes of device memory.
MIE_EXPORT int mie_mid_gemm(const void* X, long ldx, const void* W, long ldw, float* part, int M, int N, int K,
                            int wanted_splits, const void* zeros, hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 128) MIE_FAIL("mid_gemm: %d rows (at most 128)", M);
  if (K <= 0 || (K & 7)) MIE_FAIL("mid_gemm: K = %d must be a positive multiple of 8", K);
  if (ldx < K || ldw < K || (ldw & 7) || (ldx & 7)) MIE_FAIL("mid_gemm: leading dims %ld, %ld for K %d", ldx, ldw, K);
  if ((((uintptr_t)X | (uintptr_t)W | (uintptr_t)zeros) & 15) || !zeros || !part) MIE_FAIL("mid_gemm: operands must be 16-byte aligned");
  if (wanted_splits < 1 || wanted_splits > 64) MIE_FAIL("mid_gemm: %d splits", wanted_splits);
  int kper, splits;
  cut_k(K, wanted_splits, &kper, &splits);
  dim3 grid((N + 16 * MID_WAVES - 1) / (16 * MID_WAVES), splits);
  if (M <= 64) return launch_mid<4>(grid, s, (const bf16*)X, ldx, (const bf16*)W, ldw, part, M, N, K, kper, (const bf16*)zeros);
  return launch_mid<8>(grid, s, (const bf16*)X, ldx, (const bf16*)W, ldw, part, M, N, K, kper, (const bf16*)zeros);
}

// mode 0: out bfloat16 [M, ldo] = sum; 1: out float32; 2: stream [M, N] float32 += sum; 3: as 2, and
// x_next [M, ldx_next] bfloat16 = RMSNorm(stream) with weight g (bfloat16, or float32 if g_f32) and eps.
MIE_EXPORT int mie_mid_reduce(const float* part, int splits, int M, int N, int mode, void* out, long ldo, float* stream,
                              const void* g, int g_f32, void* x_next, long ldx_next, float eps, hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (splits < 1 || !part) MIE_FAIL("mid_reduce: %d splits", splits);
  if ((N & 3) || N > 4 * RED_THREADS * RED_VEC) MIE_FAIL("mid_reduce: width %d (multiples of 4 up to %d)", N, 4 * RED_THREADS * RED_VEC);
  const size_t stride = (size_t)M * N;
  dim3 grid(M), block(RED_THREADS);
  switch (mode) {
    case RED_STORE_BF16:
    case RED_STORE_F32:
      if (!out || ldo < N || (ldo & 3) || ((uintptr_t)out & 15)) MIE_FAIL("mid_reduce: output operand");
      if (mode == RED_STORE_BF16)
        hipLaunchKernelGGL(reduce_rows_kernel<RED_STORE_BF16>, grid, block, 0, s, part, splits, stride, N, out, ldo, nullptr, nullptr, 0, nullptr, 0L, 0.f);
      else
        hipLaunchKernelGGL(reduce_rows_kernel<RED_STORE_F32>, grid, block, 0, s, part, splits, stride, N, out, ldo, nullptr, nullptr, 0, nullptr, 0L, 0.f);
      break;
    case RED_ADD:
      if (!stream || ((uintptr_t)stream & 15)) MIE_FAIL("mid_reduce: stream operand");
      hipLaunchKernelGGL(reduce_rows_kernel<RED_ADD>, grid, block, 0, s, part, splits, stride, N, nullptr, 0L, stream, nullptr, 0, nullptr, 0L, 0.f);
      break;
    case RED_ADD_NORM:
      if (!stream || !g || !x_next || ldx_next < N || (ldx_next & 3) || (((uintptr_t)stream | (uintptr_t)g | (uintptr_t)x_next) & 15))
        MIE_FAIL("mid_reduce: norm operands");
      hipLaunchKernelGGL(reduce_rows_kernel<RED_ADD_NORM>, grid, block, 0, s, part, splits, stride, N, nullptr, 0L, stream, g, g_f32,
                         (bf16*)x_next, ldx_next, eps);
      break;
    default: MIE_FAIL("mid_reduce: mode %d", mode);
  }
  MIE_CHECK_LAUNCH("mid_reduce");
  return 0;
}

MIE_EXPORT int mie_mid_reduce_rope_kv(const float* part, int splits, int M, void* q_out, long ldq, const int* positions,
                                      const float* cos_t, const float* sin_t, const int* slots, void* k_cache,
                                      void* v_cache, int Hq, int Hkv, int D, int page, hipStream_t s) {
  if (M <= 0) return 0;
  if (splits < 1 || !part) MIE_FAIL("mid_reduce_rope_kv: %d splits", splits);
  if (D <= 0 || (D & 1)) MIE_FAIL("mid_reduce_rope_kv: head_dim %d", D);
  if (Hq <= 0 || Hkv <= 0 || page <= 0) MIE_FAIL("mid_reduce_rope_kv: heads %d / %d, page %d", Hq, Hkv, page);
  if (!positions || !cos_t || !sin_t || !slots || !k_cache || !v_cache || !q_out) MIE_FAIL("mid_reduce_rope_kv: null operand");
  if (ldq < (long)Hq * D) MIE_FAIL("mid_reduce_rope_kv: q leading dim %ld < %d", ldq, Hq * D);
  const size_t stride = (size_t)M * (Hq + 2 * Hkv) * D;
  hipLaunchKernelGGL(reduce_rope_kv_kernel, dim3(M, (Hq + 2 * Hkv + 3) / 4), dim3(256), 0, s, part, splits, stride, (bf16*)q_out, ldq, positions,
                     cos_t, sin_t, slots, (bf16*)k_cache, (bf16*)v_cache, Hq, Hkv, D, page);
  MIE_CHECK_LAUNCH("mid_reduce_rope_kv");
  return 0;
}
