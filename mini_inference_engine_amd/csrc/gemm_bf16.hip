// Matrix products of the bfloat16 path with few rows (M <= 64: decode steps, the head on wanted rows),
// where the weights are streamed once from HBM and everything else is noise: one kernel per product,
// with what comes before and after it folded in, because at these sizes a launch costs more than the work.
//
//   y[m, n] = sum_k x[m, k] W[n, k]          W [N, K] bfloat16 as stored in a checkpoint
//
// A workgroup of 4 or 8 waves owns 16 rows of W (one tile of C^T = W X^T); each wave streams one
// contiguous quarter (eighth) of K in 32-wide steps, the loads of the next group of steps in flight while
// the current group is multiplied; v_mfma_f32_16x16x32_bf16 with A = 16 weight rows x 32 k (16 bytes a
// lane, straight from memory) and B = 32 k x 16 batch rows; the waves' accumulators are summed through
// LDS in a fixed order.  A row's result depends on nothing but that row, K, the weights and the number of
// waves (chosen from N alone): it is bit-identical in any batch.
//
// Prologue (NORM): x is not given; instead the 32-bit residual stream r (optionally gathered rows)
//   and an RMSNorm weight g: x[m, k] = bf16(r[m, k] g[k]), the sum of r^2 is taken on the way, and the
//   result is scaled by rstd[m] = 1 / sqrt(mean(r^2) + eps) at the end (rstd is a positive scalar per row,
//   so rounding x before or after it is the same relative rounding).
// Epilogues: STORE (bfloat16 or float32 y), ADD (r[m, n] += y, the residual add of the stream, in
//   32-bit), SWIGLU (W holds gate rows then up rows; the workgroup takes the matching 16 of each and
//   writes silu(gate) * up).
#include "common.hpp"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

union Frag {
  bf16x8 v;
  uint4 q;
  uint32_t w[4];
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
  ua += 0x7FFFu + ((ua >> 16) & 1u);
  ub += 0x7FFFu + ((ub >> 16) & 1u);
  return (ua >> 16) | (ub & 0xFFFF0000u);
}

enum { EPI_STORE_BF16 = 0, EPI_STORE_F32 = 1, EPI_ADD = 2, EPI_SWIGLU = 3 };

template <int MT, bool NORM, int EPI, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
skinny_gemm_kernel(const void* __restrict__ Xv, long ldx, const int* __restrict__ rows,
                   const void* __restrict__ norm_w, int norm_w_f32, float eps, const bf16* __restrict__ W, long ldw,
                   void* __restrict__ outv, long ldo, int M, int N, int K, int up_offset) {
  constexpr int NT = EPI == EPI_SWIGLU ? 2 : 1;
  // k-steps per group of loads; with 8 waves (few tiles) each wave keeps twice as much in flight
  constexpr int U = (MT == 1 ? (NT == 2 ? 2 : 4) : (MT == 2 ? 2 : 1)) * (WAVES == 8 && !NORM ? 2 : 1);
  constexpr int SG_WAVES = WAVES;
  constexpr int SG_THREADS = WAVES * 64;
  __shared__ float s_acc[SG_WAVES][MT][256];
  __shared__ float s_ss[SG_WAVES][MT * 16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int ksteps = (K + 31) >> 5;
  const int per_wave = (ksteps + SG_WAVES - 1) / SG_WAVES;
  const int ks0 = wave * per_wave;
  const int ks1 = ks0 + per_wave < ksteps ? ks0 + per_wave : ksteps;

  // weight rows of this lane (clamped for the address; out-of-range rows are zeroed)
  const bf16* wrow[NT];
  bool wok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = n0 + col;
    wok[t] = n < N;
    wrow[t] = W + (size_t)((t ? up_offset : 0) + (wok[t] ? n : 0)) * ldw;
  }
  // batch rows of this lane
  const char* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + col;
    xok[mt] = m < M;
    const int src = xok[mt] ? (rows ? rows[m] : m) : 0;
    xrow[mt] = (const char*)Xv + (size_t)src * ldx * (NORM ? 4 : 2);
  }

  f32x4 acc[NT][MT];
  float ss[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    ss[mt] = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // One group = U k-steps.  Loads only: nothing here waits for memory, so that the next group's loads
  // stay in flight while the current group is converted and multiplied.
  struct Group {
    Frag a[U][NT];
    Frag b[U][MT];                 // !NORM: the batch fragments themselves
    float4 r[NORM ? U : 1][NORM ? MT : 1][2];   // NORM: 8 values of the stream per row and step
    uint4 g[NORM ? U : 1][2];      // NORM: 8 norm weights per step (bfloat16 in g[.][0], or float32 in both)
  };
  auto load_group = [&](Group& G, int ks) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (ks + u) * 32 + kb * 8;
      const bool kok = ks + u < ks1 && k < K;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        G.a[u][t].q = make_uint4(0, 0, 0, 0);
        if (kok && wok[t]) G.a[u][t].q = *reinterpret_cast<const uint4*>(wrow[t] + k);
      }
      if (NORM) {
        G.g[u][0] = make_uint4(0, 0, 0, 0);
        G.g[u][1] = make_uint4(0, 0, 0, 0);
        if (kok) {
          if (norm_w_f32) {
            G.g[u][0] = *reinterpret_cast<const uint4*>((const float*)norm_w + k);
            G.g[u][1] = *reinterpret_cast<const uint4*>((const float*)norm_w + k + 4);
          } else {
            G.g[u][0] = *reinterpret_cast<const uint4*>((const bf16*)norm_w + k);
          }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          G.r[u][mt][0] = make_float4(0.f, 0.f, 0.f, 0.f);
          G.r[u][mt][1] = make_float4(0.f, 0.f, 0.f, 0.f);
          if (kok && xok[mt]) {
            const float* rp = (const float*)xrow[mt] + k;
            G.r[u][mt][0] = *reinterpret_cast<const float4*>(rp);
            G.r[u][mt][1] = *reinterpret_cast<const float4*>(rp + 4);
          }
        }
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          G.b[u][mt].q = make_uint4(0, 0, 0, 0);
          if (kok && xok[mt]) G.b[u][mt].q = *reinterpret_cast<const uint4*>((const bf16*)xrow[mt] + k);
        }
      }
    }
  };
  auto multiply = [&](Group& G) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (NORM) {
        float g[8];
        if (norm_w_f32) {
          const uint32_t w8[8] = {G.g[u][0].x, G.g[u][0].y, G.g[u][0].z, G.g[u][0].w,
                                  G.g[u][1].x, G.g[u][1].y, G.g[u][1].z, G.g[u][1].w};
#pragma unroll
          for (int j = 0; j < 8; ++j) g[j] = __uint_as_float(w8[j]);
        } else {
          const uint32_t w4[4] = {G.g[u][0].x, G.g[u][0].y, G.g[u][0].z, G.g[u][0].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            g[2 * j] = __uint_as_float(w4[j] << 16);
            g[2 * j + 1] = __uint_as_float(w4[j] & 0xFFFF0000u);
          }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const float4 r0 = G.r[u][mt][0], r1 = G.r[u][mt][1];
          const float r[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
#pragma unroll
          for (int j = 0; j < 8; ++j) ss[mt] = fmaf(r[j], r[j], ss[mt]);
#pragma unroll
          for (int j = 0; j < 4; ++j) G.b[u][mt].w[j] = pack_bf16(r[2 * j] * g[2 * j], r[2 * j + 1] * g[2 * j + 1]);
        }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(G.a[u][t].v, G.b[u][mt].v, acc[t][mt], 0, 0, 0);
    }
  };

  Group g0, g1;
  load_group(g0, ks0);
  for (int ks = ks0; ks < ks1; ks += 2 * U) {
    load_group(g1, ks + U);          // in flight while group 0 is multiplied
    multiply(g0);
    load_group(g0, ks + 2 * U);
    multiply(g1);
  }

  if (NORM) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float s = ss[mt];
      s += __shfl_xor(s, 16, 64);
      s += __shfl_xor(s, 32, 64);
      if (kb == 0) s_ss[wave][mt * 16 + col] = s;
    }
  }

  // sum the waves, tile after tile, each thread owning elements (m, n) = (e / 16, e % 16)
  constexpr int PER = (MT * 256 + SG_THREADS - 1) / SG_THREADS;
  float v[NT][PER];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (t) __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) s_acc[wave][mt][lane * 4 + i] = acc[t][mt][i];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + j * SG_THREADS;
      float sum = 0.f;
      if (e < MT * 256) {
        const int mm = e >> 4, nn = e & 15;
        const int src = (((nn >> 2) << 4) + (mm & 15)) * 4 + (nn & 3);
#pragma unroll
        for (int w = 0; w < SG_WAVES; ++w) sum += s_acc[w][mm >> 4][src];
      }
      v[t][j] = sum;
    }
  }

#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = threadIdx.x + j * SG_THREADS;
    if (e >= MT * 256) continue;
    const int m = e >> 4, n = n0 + (e & 15);
    if (m >= M || n >= N) continue;
    float rstd = 1.f;
    if (NORM) {
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < SG_WAVES; ++w) tot += s_ss[w][m];
      rstd = 1.0f / sqrtf(tot / (float)K + eps);
    }
    const size_t o = (size_t)m * ldo + n;
    if (EPI == EPI_STORE_BF16) {
      ((bf16*)outv)[o] = __float2bfloat16(v[0][j] * rstd);
    } else if (EPI == EPI_STORE_F32) {
      ((float*)outv)[o] = v[0][j] * rstd;
    } else if (EPI == EPI_ADD) {
      ((float*)outv)[o] += v[0][j] * rstd;
    } else {
      const float g = v[0][j] * rstd, u = v[NT - 1][j] * rstd;
      ((bf16*)outv)[o] = __float2bfloat16(g / (1.0f + expf(-g)) * u);
    }
  }
}

MIE_EXPORT const char* gemm_bf16_last_error() { return g_mie_error; }
MIE_EXPORT int mie_skinny_max_rows() { return 64; }

template <int MT, bool NORM, int WAVES>
static int launch_epi(int epi, dim3 grid, hipStream_t s, const void* X, long ldx, const int* rows, const void* norm_w,
                      int norm_w_f32, float eps, const bf16* W, long ldw, void* out, long ldo, int M, int N, int K,
                      int up_offset) {
#define SG_LAUNCH(E)                                                                                               \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT, NORM, E, WAVES>), grid, dim3(WAVES * 64), 0, s, X, ldx, rows, norm_w, \
                     norm_w_f32, eps, W, ldw, out, ldo, M, N, K, up_offset)
  switch (epi) {
    case EPI_STORE_BF16: SG_LAUNCH(EPI_STORE_BF16); break;
    case EPI_STORE_F32: SG_LAUNCH(EPI_STORE_F32); break;
    case EPI_ADD: SG_LAUNCH(EPI_ADD); break;
    case EPI_SWIGLU: SG_LAUNCH(EPI_SWIGLU); break;
    default: MIE_FAIL("skinny_gemm: epilogue code %d", epi);
  }
#undef SG_LAUNCH
  MIE_CHECK_LAUNCH("skinny_gemm");
  return 0;
}

template <int MT, bool NORM>
static int launch_waves(int waves, int epi, dim3 grid, hipStream_t s, const void* X, long ldx, const int* rows,
                        const void* norm_w, int norm_w_f32, float eps, const bf16* W, long ldw, void* out, long ldo,
                        int M, int N, int K, int up_offset) {
  if (waves == 8) return launch_epi<MT, NORM, 8>(epi, grid, s, X, ldx, rows, norm_w, norm_w_f32, eps, W, ldw, out, ldo, M, N, K, up_offset);
  return launch_epi<MT, NORM, 4>(epi, grid, s, X, ldx, rows, norm_w, norm_w_f32, eps, W, ldw, out, ldo, M, N, K, up_offset);
}

// X: bfloat16 [M, K] (norm_w null), or the float32 stream with norm_w (RMSNorm weight, bfloat16 or float32)
// and eps.  rows: optional int32 [M] gather of X's rows.  epi: 0 bfloat16 y, 1 float32 y, 2 out[m, n] += y
// (float32), 3 silu(gate) * up with W = [gate rows (N of them); up rows] and N = the intermediate size.
MIE_EXPORT int mie_skinny_gemm(const void* X, long ldx, const int* rows, const void* norm_w, int norm_w_f32, float eps,
                               const void* W, long ldw, void* out, long ldo, int epi, int M, int N, int K,
                               hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64) MIE_FAIL("skinny_gemm: %d rows (at most 64)", M);
  if (K <= 0 || (K & 7)) MIE_FAIL("skinny_gemm: K = %d must be a positive multiple of 8", K);
  if (ldx < K || ldw < K || (ldw & 7) || (ldx & (norm_w ? 3 : 7))) MIE_FAIL("skinny_gemm: leading dims %ld, %ld for K %d", ldx, ldw, K);
  if (ldo < N) MIE_FAIL("skinny_gemm: output leading dim %ld < %d", ldo, N);
  if (((uintptr_t)X | (uintptr_t)W | (uintptr_t)norm_w) & 15) MIE_FAIL("skinny_gemm: operands must be 16-byte aligned");
  const int tiles = (N + 15) / 16;
  dim3 grid(tiles);
  const int up_offset = N;
  const bf16* Wb = (const bf16*)W;
  const int MT = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  // few tiles: more waves per tile, so that enough loads are in flight to fill the memory system
  const int waves = tiles < 256 ? 8 : 4;
  if (norm_w) {
    if (MT == 1) return launch_waves<1, true>(waves, epi, grid, s, X, ldx, rows, norm_w, norm_w_f32, eps, Wb, ldw, out, ldo, M, N, K, up_offset);
    if (MT == 2) return launch_waves<2, true>(waves, epi, grid, s, X, ldx, rows, norm_w, norm_w_f32, eps, Wb, ldw, out, ldo, M, N, K, up_offset);
    return launch_waves<4, true>(waves, epi, grid, s, X, ldx, rows, norm_w, norm_w_f32, eps, Wb, ldw, out, ldo, M, N, K, up_offset);
  }
  if (MT == 1) return launch_waves<1, false>(waves, epi, grid, s, X, ldx, rows, nullptr, 0, 0.f, Wb, ldw, out, ldo, M, N, K, up_offset);
  if (MT == 2) return launch_waves<2, false>(waves, epi, grid, s, X, ldx, rows, nullptr, 0, 0.f, Wb, ldw, out, ldo, M, N, K, up_offset);
  return launch_waves<4, false>(waves, epi, grid, s, X, ldx, rows, nullptr, 0, 0.f, Wb, ldw, out, ldo, M, N, K, up_offset);
}
