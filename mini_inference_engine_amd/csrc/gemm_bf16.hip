// Matrix products of the bfloat16 path with few rows (M <= 64: decode steps, the head on wanted rows),
// where the weights are streamed once from HBM and everything else is noise: one kernel per product,
// with what comes after it folded in, because at these sizes a launch costs as much as the work.
//
//   y[m, n] = sum_k x[m, k] W[n, k]          x [M, K], W [N, K] bfloat16 as stored in a checkpoint
//
// A workgroup of 4 or 8 waves owns 16 rows of W (one tile of C^T = W X^T); each wave streams one
// contiguous quarter (eighth) of K in 32-wide steps, two groups of steps at a time;
// v_mfma_f32_16x16x32_bf16 with A = 16 weight rows x 32 k (16 bytes a lane, straight from memory) and
// B = 32 k x 16 batch rows; the waves' accumulators are summed through LDS in a fixed order.  A row's
// result depends on nothing but that row, K, the weights and the number of waves (chosen from N alone):
// it is bit-identical in any batch.
//
// Epilogues: STORE (bfloat16 or float32 y), ADD (r[m, n] += y, the residual add of the 32-bit stream),
//   SWIGLU (W holds gate rows then up rows; the workgroup takes the matching 16 of each and writes
//   silu(gate) * up).
//   ROPE (the q/k/v projection: rotary on q and k, cache write of k and v).
// The RMSNorm between two products is folded into them as well, see NormArgs below.  (A norm prologue that
// converted the 32-bit stream inside every workgroup was measured and dropped: redoing the conversion of
// all of x per workgroup cost more than a separate norm kernel.)
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

enum { EPI_STORE_BF16 = 0, EPI_STORE_F32 = 1, EPI_ADD = 2, EPI_SWIGLU = 3, EPI_ROPE = 4 };

// What the rotary epilogue needs beside the product: W is the fused q/k/v projection; the workgroup owns
// columns j0 .. j0 + 15 and j0 + D/2 .. j0 + D/2 + 15 of one head, i.e. 16 rotary pairs.
struct RopeArgs {
  const int* positions;      // [M]
  const float* cos_t;        // [positions, D / 2]
  const float* sin_t;
  const int* slots;          // [M] cache slot of each row's token
  bf16* k_cache;             // [pages, Hkv, page, D]
  bf16* v_cache;             // [pages, Hkv, D, page]
  int Hq, Hkv, D, page;
};

// The RMSNorm between two of these products, without a kernel of its own (NF).  The product that adds
// into the stream (ADD) also writes, for the norm that follows it with weight g, x_next[m, n] =
// bf16(r[m, n] g[n]) and the sum of r[m, n]^2 over its 16 columns (ss_out [tiles, 64]); the product that
// consumes the normed value takes x_next as its X, sums ss_in over the tiles and scales its results by
// rstd[m] = 1 / sqrt(sum / width + eps): rstd is a positive scalar per row, so applying it after the
// product, to values rounded before it, is the same relative rounding as rounding the normed value.
struct NormArgs {
  const void* g;             // ADD: weight of the next norm [N]
  int g_f32;
  bf16* x_next;              // ADD: [M, ldx_next]
  long ldx_next;
  float* ss_out;             // ADD: [tiles of this product, 64]
  const float* ss_in;        // others: [ss_tiles, 64], indexed by source row
  int ss_tiles;
  float inv_width, eps;
  const int* rows;           // others: optional gather of X's (and ss_in's) rows, int32 [M]
};

template <int MT, int EPI, int WAVES, bool NF>
__global__ void __launch_bounds__(WAVES * 64)
skinny_gemm_kernel(const bf16* __restrict__ X, long ldx, const bf16* __restrict__ W, long ldw, void* __restrict__ outv,
                   long ldo, int M, int N, int K, int up_offset, RopeArgs rope, NormArgs nf) {
  constexpr int NT = (EPI == EPI_SWIGLU || EPI == EPI_ROPE) ? 2 : 1;
  // k-steps per group of loads (two groups are in flight per wave)
#ifndef SG_U_SCALE
#define SG_U_SCALE 1
#endif
  constexpr int U = (MT == 1 ? (NT == 2 ? 2 : 4) : (MT == 2 ? 2 : 1)) * SG_U_SCALE;
  constexpr int SG_WAVES = WAVES;
  constexpr int SG_THREADS = WAVES * 64;
  __shared__ float s_acc[SG_WAVES][MT][256];
  __shared__ float s_rstd[MT * 16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  int n0 = blockIdx.x * 16;
  if (EPI == EPI_ROPE) {                     // tiles are numbered per head: D / 32 pairs of tiles each
    const int per_head = rope.D >> 5;
    n0 = (blockIdx.x / per_head) * rope.D + (blockIdx.x % per_head) * 16;
  }
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
  const bf16* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + col;
    const int src = m < M ? (NF && EPI != EPI_ADD && nf.rows ? nf.rows[m] : m) : 0;
    xrow[mt] = X + (size_t)src * ldx;
  }
  // Fused norm, consuming side: the partial sums of squares are asked for here and used after the main
  // loop, so that their latency hides behind the weights'.  16 lanes a row, lane sub takes tiles sub,
  // sub + 16, ...: the first SSP of them now, the rest (widths above 4096) after the loop.
  constexpr int PER = (MT * 256 + SG_THREADS - 1) / SG_THREADS;
  constexpr int SSP = 4;
  float ssp[PER][SSP];
  if (NF && EPI != EPI_ADD) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + j * SG_THREADS;
      const int mm = (e >> 4) < MT * 16 ? (e >> 4) : 0, sub = e & 15;
      const int src = mm < M ? (nf.rows ? nf.rows[mm] : mm) : 0;
#pragma unroll
      for (int i = 0; i < SSP; ++i) {
        const int t = sub + 16 * i;
        ssp[j][i] = nf.ss_in[(size_t)(t < nf.ss_tiles ? t : 0) * 64 + src];
      }
    }
  }

  f32x4 acc[NT][MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // One group = U k-steps.  load_group only issues loads (raw values into registers) and notes which
  // steps count; the zeroing of steps that do not count happens in multiply(), so no load is waited
  // for where it is issued.
  // Every load is unconditional, from an address clamped into the operand (k 0 for steps beyond this
  // wave's range, row 0 for rows beyond M or N, whose results are never stored).
  struct Group {
    uint4 a[U][NT];
    uint4 b[U][MT];
    bool ok[U];
  };
  auto load_group = [&](Group& G, int ks) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (ks + u) * 32 + kb * 8;
      const bool kok = ks + u < ks1 && k < K;
      const int kc = kok ? k : 0;
      G.ok[u] = kok;
#pragma unroll
      for (int t = 0; t < NT; ++t) G.a[u][t] = *reinterpret_cast<const uint4*>(wrow[t] + kc);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) G.b[u][mt] = *reinterpret_cast<const uint4*>(xrow[mt] + kc);
    }
  };
  auto multiply = [&](Group& G) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool kok = G.ok[u];
      Frag a[NT], b[MT];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint4 w = G.a[u][t];
        a[t].q = make_uint4(kok ? w.x : 0u, kok ? w.y : 0u, kok ? w.z : 0u, kok ? w.w : 0u);   // a step that does not count
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[mt].q = G.b[u][mt];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t].v, b[mt].v, acc[t][mt], 0, 0, 0);
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

  if (NF && EPI != EPI_ADD) {
    // 1 / sqrt(mean of squares + eps) of every row, summed in a fixed order
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + j * SG_THREADS;
      const int mm = (e >> 4) < MT * 16 ? (e >> 4) : 0, sub = e & 15;
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < SSP; ++i) sum += sub + 16 * i < nf.ss_tiles ? ssp[j][i] : 0.f;
      if (nf.ss_tiles > 16 * SSP) {
        const int src = mm < M ? (nf.rows ? nf.rows[mm] : mm) : 0;
        for (int t = sub + 16 * SSP; t < nf.ss_tiles; t += 16) sum += nf.ss_in[(size_t)t * 64 + src];
      }
      sum += __shfl_xor(sum, 1, 64);
      sum += __shfl_xor(sum, 2, 64);
      sum += __shfl_xor(sum, 4, 64);
      sum += __shfl_xor(sum, 8, 64);
      if (sub == 0 && e < MT * 256) s_rstd[mm] = 1.0f / sqrtf(sum * nf.inv_width + nf.eps);
    }
  }

  // sum the waves, tile after tile, each thread owning elements (m, n) = (e / 16, e % 16)
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
    const int m = e >> 4, n = n0 + (e & 15);
    const bool live = e < MT * 256 && m < M && n < N;
    if (EPI == EPI_ADD) {
      const size_t o = (size_t)m * ldo + n;
      float r = 0.f;
      if (live) {
        r = ((float*)outv)[o] + v[0][j];
        ((float*)outv)[o] = r;
      }
      if (NF) {
        if (live) {
          const float g = nf.g_f32 ? ((const float*)nf.g)[n] : __bfloat162float(((const bf16*)nf.g)[n]);
          nf.x_next[(size_t)m * nf.ldx_next + n] = __float2bfloat16(r * g);
        }
        float q = r * r;                       // the 16 lanes of a row: sum of squares over this tile's columns
        q += __shfl_xor(q, 1, 64);
        q += __shfl_xor(q, 2, 64);
        q += __shfl_xor(q, 4, 64);
        q += __shfl_xor(q, 8, 64);
        if ((e & 15) == 0 && e < MT * 256 && m < M) nf.ss_out[(size_t)blockIdx.x * 64 + m] = q;
      }
      continue;
    }
    if (!live) continue;
    const float rstd = NF ? s_rstd[m] : 1.f;
    const size_t o = (size_t)m * ldo + n;
    if (EPI == EPI_ROPE) {
      const int D = rope.D, half = D >> 1;
      const int head = n / D, jd = n - head * D;         // jd < D / 2: the first of the pair
      const float x1 = v[0][j] * rstd, x2 = v[NT - 1][j] * rstd;
      if (head < rope.Hq + rope.Hkv) {
        const int pos = rope.positions[m];
        const float c = rope.cos_t[(size_t)pos * half + jd], sn = rope.sin_t[(size_t)pos * half + jd];
        const bf16 o1 = __float2bfloat16(x1 * c - x2 * sn), o2 = __float2bfloat16(x2 * c + x1 * sn);
        if (head < rope.Hq) {
          bf16* q = (bf16*)outv + (size_t)m * ldo + (size_t)head * D + jd;
          q[0] = o1;
          q[half] = o2;
        } else {
          const int slot = rope.slots[m];
          bf16* kc = rope.k_cache + (((size_t)(slot / rope.page) * rope.Hkv + (head - rope.Hq)) * rope.page +
                                     slot % rope.page) * D + jd;
          kc[0] = o1;
          kc[half] = o2;
        }
      } else {
        const int slot = rope.slots[m];
        bf16* vc = rope.v_cache + (((size_t)(slot / rope.page) * rope.Hkv + (head - rope.Hq - rope.Hkv)) * D + jd) *
                                      rope.page + slot % rope.page;
        vc[0] = __float2bfloat16(x1);
        vc[(size_t)half * rope.page] = __float2bfloat16(x2);
      }
    } else if (EPI == EPI_STORE_BF16) {
      ((bf16*)outv)[o] = __float2bfloat16(v[0][j] * rstd);
    } else if (EPI == EPI_STORE_F32) {
      ((float*)outv)[o] = v[0][j] * rstd;
    } else {
      const float g = v[0][j] * rstd, u = v[NT - 1][j] * rstd;
      ((bf16*)outv)[o] = __float2bfloat16(g / (1.0f + expf(-g)) * u);
    }
  }
}

MIE_EXPORT const char* gemm_bf16_last_error() { return g_mie_error; }
MIE_EXPORT int mie_skinny_max_rows() { return 64; }

template <int MT, int WAVES, bool NF>
static int launch_epi(int epi, dim3 grid, hipStream_t s, const bf16* X, long ldx, const bf16* W, long ldw, void* out,
                      long ldo, int M, int N, int K, int up_offset, const RopeArgs& rope, const NormArgs& nf) {
#define SG_LAUNCH(E)                                                                                               \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT, E, WAVES, NF>), grid, dim3(WAVES * 64), 0, s, X, ldx, W, ldw, out, ldo, M, \
                     N, K, up_offset, rope, nf)
  switch (epi) {
    case EPI_STORE_BF16: SG_LAUNCH(EPI_STORE_BF16); break;
    case EPI_STORE_F32: SG_LAUNCH(EPI_STORE_F32); break;
    case EPI_ADD: SG_LAUNCH(EPI_ADD); break;
    case EPI_SWIGLU: SG_LAUNCH(EPI_SWIGLU); break;
    case EPI_ROPE: SG_LAUNCH(EPI_ROPE); break;
    default: MIE_FAIL("skinny_gemm: epilogue code %d", epi);
  }
#undef SG_LAUNCH
  MIE_CHECK_LAUNCH("skinny_gemm");
  return 0;
}

template <int MT>
static int launch_waves(int waves, bool fused_norm, int epi, dim3 grid, hipStream_t s, const bf16* X, long ldx,
                        const bf16* W, long ldw, void* out, long ldo, int M, int N, int K, int up_offset,
                        const RopeArgs& rope, const NormArgs& nf) {
  if (fused_norm) {
    if (waves == 8) return launch_epi<MT, 8, true>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, nf);
    return launch_epi<MT, 4, true>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, nf);
  }
  if (waves == 8) return launch_epi<MT, 8, false>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, nf);
  return launch_epi<MT, 4, false>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, nf);
}

static int launch_rows(int tiles, int epi, hipStream_t s, const bf16* X, long ldx, const bf16* W, long ldw, void* out,
                       long ldo, int M, int N, int K, int up_offset, const RopeArgs& rope, const NormArgs* nf) {
  dim3 grid(tiles);
  const int MT = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  // few tiles: more waves per tile, so that enough loads are in flight to fill the memory system
  const int waves = tiles < 256 ? 8 : 4;
  NormArgs none = {};
  const NormArgs& n = nf ? *nf : none;
  if (MT == 1) return launch_waves<1>(waves, nf != nullptr, epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, n);
  if (MT == 2) return launch_waves<2>(waves, nf != nullptr, epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, n);
  return launch_waves<4>(waves, nf != nullptr, epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, n);
}

static int check_operands(const char* what, const void* X, long ldx, const void* W, long ldw, int M, int K) {
  if (M > 64) MIE_FAIL("%s: %d rows (at most 64)", what, M);
  if (K <= 0 || (K & 7)) MIE_FAIL("%s: K = %d must be a positive multiple of 8", what, K);
  if (ldx < K || ldw < K || (ldw & 7) || (ldx & 7)) MIE_FAIL("%s: leading dims %ld, %ld for K %d", what, ldx, ldw, K);
  if (((uintptr_t)X | (uintptr_t)W) & 15) MIE_FAIL("%s: operands must be 16-byte aligned", what);
  return 0;
}

// The fused norm, both sides.  Producer (epi 2 only): next_g (weight of the norm that follows, bfloat16 or
// float32), x_next [M, ldx_next] bfloat16 and ss_out [ceil(N / 16), 64] float32 are written beside the add.
// Consumer (other epilogues): X is a producer's x_next, ss_in its ss_out with ss_tiles tiles, width the
// norm's width (= K), rows an optional int32 [M] gather of X's rows.  Pass ss_in = next_g = null for none.
static int fill_norm_args(NormArgs& nf, int epi, const void* next_g, int next_g_f32, void* x_next, long ldx_next,
                          float* ss_out, const float* ss_in, int ss_tiles, int width, float eps, const int* rows,
                          int N) {
  nf = NormArgs{};
  if (epi == EPI_ADD) {
    if (!next_g || !x_next || !ss_out || ldx_next < N) MIE_FAIL("skinny_gemm: fused norm output operands");
    nf.g = next_g; nf.g_f32 = next_g_f32; nf.x_next = (bf16*)x_next; nf.ldx_next = ldx_next; nf.ss_out = ss_out;
  } else {
    if (!ss_in || ss_tiles <= 0 || width <= 0) MIE_FAIL("skinny_gemm: fused norm input operands");
    nf.ss_in = ss_in; nf.ss_tiles = ss_tiles; nf.inv_width = 1.0f / (float)width; nf.eps = eps; nf.rows = rows;
  }
  return 0;
}

// X [M, K] and W bfloat16.  epi: 0 bfloat16 y, 1 float32 y, 2 out[m, n] += y (float32), 3 silu(gate) * up with
// W = [gate rows (N of them); up rows] and N = the intermediate size.
MIE_EXPORT int mie_skinny_gemm(const void* X, long ldx, const void* W, long ldw, void* out, long ldo, int epi, int M,
                               int N, int K, const void* next_g, int next_g_f32, void* x_next, long ldx_next,
                               float* ss_out, const float* ss_in, int ss_tiles, float eps, const int* rows,
                               hipStream_t s) {
  if (M <= 0 || N <= 0) return 0;
  if (epi < 0 || epi > EPI_SWIGLU) MIE_FAIL("skinny_gemm: epilogue code %d", epi);
  if (check_operands("skinny_gemm", X, ldx, W, ldw, M, K)) return -1;
  if (ldo < N) MIE_FAIL("skinny_gemm: output leading dim %ld < %d", ldo, N);
  RopeArgs none = {};
  NormArgs nf;
  const bool fused = next_g || ss_in;
  if (fused && fill_norm_args(nf, epi, next_g, next_g_f32, x_next, ldx_next, ss_out, ss_in, ss_tiles, K, eps, rows, N)) return -1;
  if (!fused && rows) MIE_FAIL("skinny_gemm: a row gather comes with the fused norm only");
  return launch_rows((N + 15) / 16, epi, s, (const bf16*)X, ldx, (const bf16*)W, ldw, out, ldo, M, N, K, N, none,
                     fused ? &nf : nullptr);
}

// The fused q/k/v projection of single-token rows with what follows it: W [(Hq + 2 Hkv) D, K]; rotary
// (half-split pairs over the whole head, angles from cos/sin [positions, D / 2] float32) on the q and k
// heads in 32-bit, q [M, Hq D] written to q_out, rotated k and v written to cache slot slots[m]
// (k_cache [pages, Hkv, page, D], v_cache [pages, Hkv, D, page]).  D must be a multiple of 32.
// With ss_in: X is a fused-norm producer's x_next (see above).
MIE_EXPORT int mie_skinny_qkv_rope(const void* X, long ldx, const void* W, long ldw, void* q_out, long ldq,
                                   const int* positions, const float* cos_t, const float* sin_t, const int* slots,
                                   void* k_cache, void* v_cache, int M, int Hq, int Hkv, int D, int page, int K,
                                   const float* ss_in, int ss_tiles, float eps, hipStream_t s) {
  if (M <= 0) return 0;
  if (D <= 0 || (D & 31)) MIE_FAIL("skinny_qkv_rope: head_dim %d must be a multiple of 32", D);
  if (Hq <= 0 || Hkv <= 0 || page <= 0) MIE_FAIL("skinny_qkv_rope: heads %d / %d, page %d", Hq, Hkv, page);
  if (!positions || !cos_t || !sin_t || !slots || !k_cache || !v_cache || !q_out) MIE_FAIL("skinny_qkv_rope: null operand");
  if (check_operands("skinny_qkv_rope", X, ldx, W, ldw, M, K)) return -1;
  if (ldq < (long)Hq * D) MIE_FAIL("skinny_qkv_rope: q leading dim %ld < %d", ldq, Hq * D);
  RopeArgs rope = {positions, cos_t, sin_t, slots, (bf16*)k_cache, (bf16*)v_cache, Hq, Hkv, D, page};
  const int heads = Hq + 2 * Hkv;
  NormArgs nf;
  if (ss_in && fill_norm_args(nf, EPI_ROPE, nullptr, 0, nullptr, 0, nullptr, ss_in, ss_tiles, K, eps, nullptr, heads * D)) return -1;
  return launch_rows(heads * (D / 32), EPI_ROPE, s, (const bf16*)X, ldx, (const bf16*)W, ldw, q_out, ldq, M, heads * D, K,
                     D / 2, rope, ss_in ? &nf : nullptr);
}
