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
//   SWIGLU (W holds gate rows then up rows; a tile is 8 gate rows and the matching 8 up rows, and the
//   workgroup writes silu(gate) * up for them).
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
// columns j0 .. j0 + 7 and j0 + D/2 .. j0 + D/2 + 7 of one head, i.e. 8 rotary pairs.
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
// bf16(r[m, n] g[n]) and the sum of r[m, n]^2 over its 16 columns (ss_out [M, tiles]); the product that
// consumes the normed value takes x_next as its X, sums ss_in over the tiles and scales its results by
// rstd[m] = 1 / sqrt(sum / width + eps): rstd is a positive scalar per row, so applying it after the
// product, to values rounded before it, is the same relative rounding as rounding the normed value.
struct NormArgs {
  const void* g;             // ADD: weight of the next norm [N]
  int g_f32;
  bf16* x_next;              // ADD: [M, ldx_next]
  long ldx_next;
  float* ss_out;             // ADD: [M, tiles of this product rounded up to a multiple of 4]
  const float* ss_in;        // others: [rows, ss_tiles rounded up to a multiple of 4], indexed by source row
  int ss_tiles;
  float inv_width, eps;
  const int* rows;           // others: optional gather of X's (and ss_in's) rows, int32 [M]
};

// Which weight row column c (0 .. 15) of tile `tile` multiplies, and whether it exists.
//   plain:  n = 16 tile + c
//   SWIGLU: columns 0 .. 7 are gate rows j = 8 tile + c, columns 8 .. 15 the up rows of the same j
//   ROPE:   columns 0 .. 7 are the first members jd = 8 (tile % (D / 16)) + c of eight rotary pairs of head
//           tile / (D / 16), columns 8 .. 15 their partners jd + D / 2
// so that both members of a pair are lanes c and c ^ 8 of one wave after the reduction.
template <int EPI>
__device__ __forceinline__ long tile_column(int tile, int c, int N, int up_offset, int D, bool& ok) {
  if (EPI == EPI_SWIGLU) {
    const int j = tile * 8 + (c & 7);
    ok = j < N;
    return (long)(c >> 3) * up_offset + j;
  }
  if (EPI == EPI_ROPE) {
    const int per_head = D >> 4, head = tile / per_head, jd = (tile - head * per_head) * 8 + (c & 7);
    ok = true;
    return (long)head * D + jd + (c >> 3) * (D >> 1);
  }
  const int n = tile * 16 + c;
  ok = n < N;
  return n;
}

template <int MT, int EPI, int WAVES, bool NF>
__global__ void __launch_bounds__(WAVES * 64)
skinny_gemm_kernel(const bf16* __restrict__ X, long ldx, const bf16* __restrict__ W, long ldw, void* __restrict__ outv,
                   long ldo, int M, int N, int K, int up_offset, RopeArgs rope, NormArgs nf) {
  // k-steps per group of loads (two groups are in flight per wave)
  constexpr int U = MT == 1 ? 4 : 2;
  constexpr int SG_WAVES = WAVES;
  constexpr int SG_THREADS = WAVES * 64;
  constexpr int PER = (MT * 256 + SG_THREADS - 1) / SG_THREADS;   // results (m, n) a thread owns after the reduction
  __shared__ float s_acc[SG_WAVES][MT][256];
  __shared__ float s_rstd[MT * 16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int tile = blockIdx.x;
  const int ksteps = (K + 31) >> 5;
  const int per_wave = (ksteps + SG_WAVES - 1) / SG_WAVES;
  const int ks0 = wave * per_wave;
  const int ks1 = ks0 + per_wave < ksteps ? ks0 + per_wave : ksteps;

  // What the epilogue reads beside the product is asked for first, so that it has arrived long before it is used.
  float e_old[PER], e_cos[PER], e_sin[PER];
  uint32_t e_g[PER];                       // raw bits of the next norm's weight (converted where it is used)
  int e_slot[PER], e_pos[PER];
  bool e_live[PER];
  long e_n[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = threadIdx.x + j * SG_THREADS;
    const int m = e >> 4;
    bool ok;
    e_n[j] = tile_column<EPI>(tile, e & 15, N, up_offset, rope.D, ok);
    e_live[j] = e < MT * 256 && m < M && ok;
    // every load below is unconditional, from an address clamped into the operand
    const int mc = e_live[j] ? m : 0;
    const long nc = e_live[j] ? e_n[j] : 0;
    e_old[j] = e_cos[j] = e_sin[j] = 0.f;
    e_g[j] = 0u;
    e_slot[j] = e_pos[j] = 0;
    if (EPI == EPI_ADD) {
      e_old[j] = ((const float*)outv)[(size_t)mc * ldo + nc];
      if (NF) e_g[j] = nf.g_f32 ? ((const uint32_t*)nf.g)[nc] : (uint32_t)((const uint16_t*)nf.g)[nc];
    }
    if (EPI == EPI_ROPE) {
      e_pos[j] = rope.positions[mc];
      e_slot[j] = rope.slots[mc];
    }
  }
  // Fused norm, consuming side: the partial sums of squares likewise.  16 lanes a row, lane sub takes
  // the tiles 4 (sub + 16 i) .. + 3: the first SSP fours now, the rest (widths above 4096) after the loop.
  constexpr int SSP = 4;
  float4 ssp[PER][SSP];
  const int ss_ld = (nf.ss_tiles + 3) & ~3;
  if (NF && EPI != EPI_ADD) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + j * SG_THREADS;
      const int mm = (e >> 4) < MT * 16 ? (e >> 4) : 0, sub = e & 15;
      const int src = mm < M ? (nf.rows ? nf.rows[mm] : mm) : 0;
#pragma unroll
      for (int i = 0; i < SSP; ++i) {
        const int t = 4 * (sub + 16 * i);
        ssp[j][i] = *reinterpret_cast<const float4*>(nf.ss_in + (size_t)src * ss_ld + (t < ss_ld ? t : 0));
      }
    }
  }

  // weight row of this lane (clamped for the address; a row that does not exist is never stored)
  bool wok;
  const long wr = tile_column<EPI>(tile, col, N, up_offset, rope.D, wok);
  const bf16* wrow = W + (size_t)(wok ? wr : 0) * ldw;
  // batch rows of this lane; lanes of rows beyond M read row 0 along with the lanes that own it
  const bf16* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + col;
    const int src = m < M ? (NF && EPI != EPI_ADD && nf.rows ? nf.rows[m] : m) : 0;
    xrow[mt] = X + (size_t)src * ldx;
  }

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // One group = U k-steps.  load_group only issues loads (raw values into registers) and notes which
  // steps count; the zeroing of steps that do not count happens in multiply(), so no load is waited
  // for where it is issued.  Every load is unconditional, from an address clamped into the operand
  // (k 0 for steps beyond this wave's range).
  struct Group {
    uint4 a[U];
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
      G.a[u] = *reinterpret_cast<const uint4*>(wrow + kc);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) G.b[u][mt] = *reinterpret_cast<const uint4*>(xrow[mt] + kc);
    }
  };
  auto multiply = [&](Group& G) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool kok = G.ok[u];
      Frag a, b[MT];
      const uint4 w = G.a[u];
      a.q = make_uint4(kok ? w.x : 0u, kok ? w.y : 0u, kok ? w.z : 0u, kok ? w.w : 0u);   // a step that does not count
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[mt].q = G.b[u][mt];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b[mt].v, acc[mt], 0, 0, 0);
    }
  };

  Group g0, g1;
  load_group(g0, ks0);
  if (EPI == EPI_ROPE) {
    // the angles, once the positions are here (they were asked for before the first group)
    const int half = rope.D >> 1;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + j * SG_THREADS;
      const int per_head = rope.D >> 4;
      const int jd = (tile % per_head) * 8 + (e & 7);
      e_cos[j] = rope.cos_t[(size_t)e_pos[j] * half + jd];       // position 0 for the rows that do not count
      e_sin[j] = rope.sin_t[(size_t)e_pos[j] * half + jd];
    }
  }
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
      for (int i = 0; i < SSP; ++i) {
        const int t = 4 * (sub + 16 * i);
        sum += (t < nf.ss_tiles ? ssp[j][i].x : 0.f) + (t + 1 < nf.ss_tiles ? ssp[j][i].y : 0.f) +
               (t + 2 < nf.ss_tiles ? ssp[j][i].z : 0.f) + (t + 3 < nf.ss_tiles ? ssp[j][i].w : 0.f);
      }
      if (nf.ss_tiles > 64 * SSP) {
        const int src = mm < M ? (nf.rows ? nf.rows[mm] : mm) : 0;
        for (int t = 64 * SSP + sub; t < nf.ss_tiles; t += 16) sum += nf.ss_in[(size_t)src * ss_ld + t];
      }
      sum += __shfl_xor(sum, 1, 64);
      sum += __shfl_xor(sum, 2, 64);
      sum += __shfl_xor(sum, 4, 64);
      sum += __shfl_xor(sum, 8, 64);
      if (sub == 0 && e < MT * 256) s_rstd[mm] = 1.0f / sqrtf(sum * nf.inv_width + nf.eps);
    }
  }

  // sum the waves, each thread owning elements (m, c) = (e / 16, e % 16)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) s_acc[wave][mt][lane * 4 + i] = acc[mt][i];
  __syncthreads();
  float v[PER];
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
    v[j] = sum;
  }

#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = threadIdx.x + j * SG_THREADS;
    const int m = e >> 4, c = e & 15;
    const bool live = e_live[j];
    const long n = e_n[j];
    if (EPI == EPI_ADD) {
      const float r = e_old[j] + v[j];
      if (live) ((float*)outv)[(size_t)m * ldo + n] = r;
      if (NF) {
        const float g = nf.g_f32 ? __uint_as_float(e_g[j]) : __uint_as_float(e_g[j] << 16);
        if (live) nf.x_next[(size_t)m * nf.ldx_next + n] = __float2bfloat16(r * g);
        float q = live ? r * r : 0.f;          // the 16 lanes of a row: sum of squares over this tile's columns
        q += __shfl_xor(q, 1, 64);
        q += __shfl_xor(q, 2, 64);
        q += __shfl_xor(q, 4, 64);
        q += __shfl_xor(q, 8, 64);
        if (c == 0 && e < MT * 256 && m < M) nf.ss_out[(size_t)m * ((gridDim.x + 3) & ~3) + tile] = q;
      }
      continue;
    }
    const float rstd = NF ? s_rstd[m < MT * 16 ? m : 0] : 1.f;
    const float mine = v[j] * rstd;
    float other = 0.f;
    if (EPI == EPI_ROPE || EPI == EPI_SWIGLU) other = __shfl_xor(mine, 8, 64);   // the pair's other member
    if (!live) continue;
    if (EPI == EPI_ROPE) {
      const int D = rope.D;
      const int head = (int)(n / D), jd = (int)(n - (long)head * D);   // column inside the head
      const int slot = e_slot[j];
      if (head < rope.Hq + rope.Hkv) {
        // first member (c < 8): x1 cos - x2 sin; second: x2 cos + x1 sin, x1 being the first member's value
        const float o = c < 8 ? mine * e_cos[j] - other * e_sin[j] : mine * e_cos[j] + other * e_sin[j];
        if (head < rope.Hq)
          ((bf16*)outv)[(size_t)m * ldo + n] = __float2bfloat16(o);
        else
          rope.k_cache[(((size_t)(slot / rope.page) * rope.Hkv + (head - rope.Hq)) * rope.page + slot % rope.page) * D + jd] =
              __float2bfloat16(o);
      } else {
        rope.v_cache[(((size_t)(slot / rope.page) * rope.Hkv + (head - rope.Hq - rope.Hkv)) * D + jd) * rope.page +
                     slot % rope.page] = __float2bfloat16(mine);
      }
    } else if (EPI == EPI_STORE_BF16) {
      ((bf16*)outv)[(size_t)m * ldo + n] = __float2bfloat16(mine);
    } else if (EPI == EPI_STORE_F32) {
      ((float*)outv)[(size_t)m * ldo + n] = mine;
    } else if (c < 8) {                        // SWIGLU: mine = gate, other = up
      ((bf16*)outv)[(size_t)m * ldo + n] = __float2bfloat16(mine / (1.0f + expf(-mine)) * other);
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
#define SG_WAVES_CASE(WV)                                                                                              \
  if (waves == WV)                                                                                                     \
    return fused_norm ? launch_epi<MT, WV, true>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, nf) \
                      : launch_epi<MT, WV, false>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, nf)
  SG_WAVES_CASE(8);
  SG_WAVES_CASE(4);
#undef SG_WAVES_CASE
  MIE_FAIL("skinny_gemm: %d waves", waves);
}

// Waves a tile: the fewer tiles a product has, the more waves share one, so that enough loads are in
// flight to fill the memory system (16 waves were measured slower than 8 at every shape).  Chosen from
// the weight's shape alone, never from the batch.
static int waves_for(int tiles) { return tiles < 256 ? 8 : 4; }

static int launch_rows(int tiles, int epi, hipStream_t s, const bf16* X, long ldx, const bf16* W, long ldw, void* out,
                       long ldo, int M, int N, int K, int up_offset, const RopeArgs& rope, const NormArgs* nf) {
  dim3 grid(tiles);
  const int MT = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int waves = waves_for(tiles);
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
// float32), x_next [M, ldx_next] bfloat16 and ss_out [M, ceil(N / 16) rounded up to a multiple of 4] float32
// (16-byte aligned) are written beside the add.
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
  return launch_rows(epi == EPI_SWIGLU ? (N + 7) / 8 : (N + 15) / 16, epi, s, (const bf16*)X, ldx, (const bf16*)W, ldw, out, ldo, M, N, K, N, none,
                     fused ? &nf : nullptr);
}

// The fused q/k/v projection of single-token rows with what follows it: W [(Hq + 2 Hkv) D, K]; rotary
// (half-split pairs over the whole head, angles from cos/sin [positions, D / 2] float32) on the q and k
// heads in 32-bit, q [M, Hq D] written to q_out, rotated k and v written to cache slot slots[m]
// (k_cache [pages, Hkv, page, D], v_cache [pages, Hkv, D, page]).  D must be a multiple of 16.
// With ss_in: X is a fused-norm producer's x_next (see above).
MIE_EXPORT int mie_skinny_qkv_rope(const void* X, long ldx, const void* W, long ldw, void* q_out, long ldq,
                                   const int* positions, const float* cos_t, const float* sin_t, const int* slots,
                                   void* k_cache, void* v_cache, int M, int Hq, int Hkv, int D, int page, int K,
                                   const float* ss_in, int ss_tiles, float eps, hipStream_t s) {
  if (M <= 0) return 0;
  if (D <= 0 || (D & 15)) MIE_FAIL("skinny_qkv_rope: head_dim %d must be a multiple of 16", D);
  if (Hq <= 0 || Hkv <= 0 || page <= 0) MIE_FAIL("skinny_qkv_rope: heads %d / %d, page %d", Hq, Hkv, page);
  if (!positions || !cos_t || !sin_t || !slots || !k_cache || !v_cache || !q_out) MIE_FAIL("skinny_qkv_rope: null operand");
  if (check_operands("skinny_qkv_rope", X, ldx, W, ldw, M, K)) return -1;
  if (ldq < (long)Hq * D) MIE_FAIL("skinny_qkv_rope: q leading dim %ld < %d", ldq, Hq * D);
  RopeArgs rope = {positions, cos_t, sin_t, slots, (bf16*)k_cache, (bf16*)v_cache, Hq, Hkv, D, page};
  const int heads = Hq + 2 * Hkv;
  NormArgs nf;
  if (ss_in && fill_norm_args(nf, EPI_ROPE, nullptr, 0, nullptr, 0, nullptr, ss_in, ss_tiles, K, eps, nullptr, heads * D)) return -1;
  return launch_rows(heads * (D / 16), EPI_ROPE, s, (const bf16*)X, ldx, (const bf16*)W, ldw, q_out, ldq, M, heads * D, K,
                     D / 2, rope, ss_in ? &nf : nullptr);
}
