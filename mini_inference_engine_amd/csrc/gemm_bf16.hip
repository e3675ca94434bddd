// Matrix products of the bfloat16 path with few rows (M <= 16: decode steps, the head on wanted rows),
// where the weights are streamed once from HBM and everything else is noise: one kernel per product,
// with what comes after it folded in, because at these sizes a launch costs as much as the work.
//
//   y[m, n] = sum_k x[m, k] W[n, k]          x [M, K], W [N, K] bfloat16 as stored in a checkpoint
//
// A workgroup of 4 waves owns 16 rows of W (one tile of C^T = W X^T); each wave streams one contiguous
// quarter of K in 32-wide steps; v_mfma_f32_16x16x32_bf16 with A = 16 weight rows x 32 k and B = 32 k x 16
// batch rows; the waves' accumulators are summed through LDS in a fixed order.  A row's result depends on
// nothing but that row, K and the weights: it is bit-identical in any batch.
//
// How the operands reach the matrix instruction.  The instruction wants lane 16 b + r to hold k-block b (8
// values, 16 bytes) of row r.  Loaded in that order, a quarter wave (16 lanes) touches 16 cache lines for 16
// bytes each, and the address unit, which looks lines up one at a time, is then what bounds the kernel: the x
// loads alone (all of them hits) cost a seventh to a third of its time, and the weights stream at 4.2 to
// 4.7 TB/s where a plain read of the same bytes runs at 5.4 to 5.8.  So the loads are issued in the order lane
// 4 r + b (a quarter wave reads 64 contiguous bytes of 4 rows) and write the wave's own piece of the LDS
// directly (no registers, nothing the compiler waits for): a ring of slots of two k-steps, all but one on their
// way while that one is multiplied.  Within a row the four blocks are permuted (block b at 16-byte slot
// 4 r + (b ^ (r / 4) % 4)), so that the fragment reads (lane 16 b + r) are spread over all banks.  No barrier
// in the loop: a wave reads only what it brought in itself.  (The same order with nontemporal loads reads a
// fifth faster still when nothing else is loaded, but slower beside the x loads: measured, not used.)
//
// Epilogues: STORE (bfloat16 or float32 y), ADD (r[m, n] += y, the residual add of the 32-bit stream),
//   SWIGLU (W holds gate rows then up rows; a tile is 8 gate rows and the matching 8 up rows, and the
//   workgroup writes silu(gate) * up for them).
//   ROPE (the q/k/v projection: rotary on q and k, cache write of k and v).
// The RMSNorm between two products is folded into them as well, see NormArgs below.  (A norm prologue that
// converted the 32-bit stream inside every workgroup was measured and dropped: redoing the conversion of
// all of x per workgroup cost more than a separate norm kernel.)
#include "common.hpp"
#include <mutex>
#include <set>
#include <utility>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// what a k-step beyond a wave's range or beyond K loads instead of weights, so that every load is unconditional
__device__ __align__(64) const uint32_t mie_zero_words[16] = {0};

// wait until at most n vector memory loads of this wave are still on their way
#define SG_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

constexpr int SG_WAVES = 4;       // waves a workgroup
constexpr int SG_THREADS = SG_WAVES * 64;
constexpr int RING_U = 2;         // k-steps a slot of a wave's ring

// The fragments of a slot (U k-steps: weight fragment, x fragment, 1 KB each) out of the LDS, read and waited for
// in one piece of assembly: the compiler knows nothing of the loads that write the LDS, so a read it could see
// would make it wait for every load on its way, and it must never see a register whose value is still to arrive.
typedef uint32_t sg_u32x4 __attribute__((ext_vector_type(4)));
template <int U> struct RingRead;
template <> struct RingRead<2> {
  static __device__ __forceinline__ void run(uint32_t at, sg_u32x4 (&f)[4]) {
    asm volatile(
      "ds_read_b128 %0, %4\n\t"
      "ds_read_b128 %1, %4 offset:1024\n\t"
      "ds_read_b128 %2, %4 offset:2048\n\t"
      "ds_read_b128 %3, %4 offset:3072\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(f[0]), "=&v"(f[1]), "=&v"(f[2]), "=&v"(f[3])
      : "v"(at)
      : "memory");
  }
};

// The wait of round `it` < SLOTS - 1 (the counter's limit must be a constant of the instruction).
template <int SLOTS, int IT> struct RingStart {
  static __device__ __forceinline__ void wait(int it) {
    if (it == IT) SG_VMCNT((SLOTS - 2 - IT) * RING_U + (IT + 1) * RING_U * 2);
    else if constexpr (IT + 1 < SLOTS - 1) RingStart<SLOTS, IT + 1>::wait(it);
  }
};

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

template <int EPI, bool NF, int SLOTS>
__global__ void __launch_bounds__(SG_THREADS)
skinny_gemm_kernel(const bf16* __restrict__ X, long ldx, const bf16* __restrict__ W, long ldw, void* __restrict__ outv,
                   long ldo, int M, int N, int K, int up_offset, RopeArgs rope, NormArgs nf) {
  constexpr int SLOT_BYTES = RING_U * 2 * 1024;            // a k-step: the weight fragment, then the x fragment, 1 KB each
  constexpr int WAVE_BYTES = SLOTS * SLOT_BYTES;
  constexpr int L = RING_U * 2;                            // loads a slot
  static_assert((SLOTS - 1) * L <= 63, "more loads in flight than the counter holds");
  extern __shared__ __align__(16) char ring_lds[];         // WAVE_BYTES a wave
  __shared__ float s_acc[SG_WAVES][256];
  __shared__ float s_rstd[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int tile = blockIdx.x;
  const int ksteps = (K + 31) >> 5;
  const int per_wave = (ksteps + SG_WAVES - 1) / SG_WAVES;
  const int ks0 = wave * per_wave;
  const int ks1 = ks0 + per_wave < ksteps ? ks0 + per_wave : ksteps;

  // What this lane brings in: row lrow (of the weight tile; of x), k-block lkb of every k-step.  And the one
  // result this thread owns after the waves are summed: x row m, column c of the tile.  The gather of x's
  // rows, if there is one, and the positions are the first things asked for: addresses depend on them.
  const int lrow = lane >> 2, lkb = (lane & 3) ^ ((lrow >> 2) & 3);
  const int m = threadIdx.x >> 4, c = threadIdx.x & 15;
  const bool gather = NF && EPI != EPI_ADD && nf.rows;
  const int lsrc = lrow < M ? (gather ? nf.rows[lrow] : lrow) : 0;
  const int msrc = m < M ? (gather ? nf.rows[m] : m) : 0;

  bool ok;
  const long n = tile_column<EPI>(tile, c, N, up_offset, rope.D, ok);
  const bool live = m < M && ok;
  const int mc = live ? m : 0;
  const long nc = live ? n : 0;
  float e_old = 0.f, e_cos = 0.f, e_sin = 0.f;
  uint32_t e_g = 0u;                       // raw bits of the next norm's weight (converted where it is used)
  int e_slot = 0, e_pos = 0;
  if (EPI == EPI_ROPE) {                   // the positions: further addresses depend on them too
    e_pos = rope.positions[mc];
    e_slot = rope.slots[mc];
  }

  // The ring.  Slots beyond the wave's range load zeros only, so that it is always filled and drained the
  // same way.
  bool lok;
  const long lwr = tile_column<EPI>(tile, lrow, N, up_offset, rope.D, lok);
  const bf16* wsrc = W + (size_t)(lok ? lwr : 0) * ldw + lkb * 8;   // a row that does not exist is never stored
  const bf16* xsrc = X + (size_t)lsrc * ldx + lkb * 8;              // rows beyond M read row 0 along with the lanes that own it
  const bf16* zero_lane = reinterpret_cast<const bf16*>(mie_zero_words) + lkb * 8;   // per lane, so that choosing it is a select
  char* mine = ring_lds + wave * WAVE_BYTES;
  // what: 1 the weight fragments of slot s, 2 the x fragments, 3 both (weight, x, weight, x)
  auto issue = [&](int s, int what) {
    char* base = mine + (s % SLOTS) * SLOT_BYTES;
    const int ks = ks0 + s * RING_U;
#pragma unroll
    for (int u = 0; u < RING_U; ++u) {
      const bool kok = ks + u < ks1 && (ks + u) * 32 + lkb * 8 < K;
      const bf16* a = kok ? wsrc + (size_t)(ks + u) * 32 : zero_lane;
      const bf16* b = kok ? xsrc + (size_t)(ks + u) * 32 : zero_lane;
      if (what & 1)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)a,
                                         (__attribute__((address_space(3))) void*)(base + (2 * u) * 1024), 16, 0, 0);
      if (what & 2)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)b,
                                         (__attribute__((address_space(3))) void*)(base + (2 * u + 1) * 1024), 16, 0, 0);
    }
  };
  const int rounds = ks1 > ks0 ? (ks1 - ks0 + RING_U - 1) / RING_U : 0;
  // this lane's piece of a fragment: row col, block kb
  const uint32_t at0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)mine + (col * 4 + (kb ^ ((col >> 2) & 3))) * 16;
  // The ring starts with the weights of its first slots; their x follows below, after what the epilogue reads
  // has been asked for: all that waits for the row numbers of a gather, the weights do not.
#pragma unroll
  for (int s = 0; s < SLOTS - 1; ++s) issue(s, 1);
  // What the epilogue reads beside the product is asked for next, so that it has arrived long before it is
  // used and is older than the ring's x loads (the counter of loads on their way runs in issue order).
  // Every load is unconditional, from an address clamped into the operand.
  if (EPI == EPI_ADD) {
    e_old = ((const float*)outv)[(size_t)mc * ldo + nc];
    if (NF) e_g = nf.g_f32 ? ((const uint32_t*)nf.g)[nc] : (uint32_t)((const uint16_t*)nf.g)[nc];
  }
  // Fused norm, consuming side: the partial sums of squares likewise.  16 lanes a row, lane c takes the
  // tiles 4 (c + 16 i) .. + 3: the first SSP fours now, the rest (widths above 4096) after the loop.
  constexpr int SSP = 4;
  float4 ssp[SSP];
  const int ss_ld = (nf.ss_tiles + 3) & ~3;
  if (NF && EPI != EPI_ADD) {
#pragma unroll
    for (int i = 0; i < SSP; ++i) {
      const int t = 4 * (c + 16 * i);
      ssp[i] = *reinterpret_cast<const float4*>(nf.ss_in + (size_t)msrc * ss_ld + (t < ss_ld ? t : 0));
    }
  }

  // the x fragments of the ring's first slots
#pragma unroll
  for (int s = 0; s < SLOTS - 1; ++s) issue(s, 2);
  if (EPI == EPI_ROPE) {
    // the angles, once the positions are here (asked for before the ring: waiting for them does not wait for it)
    const int half = rope.D >> 1;
    const int per_head = rope.D >> 4;
    const int jd = (tile % per_head) * 8 + (c & 7);
    e_cos = rope.cos_t[(size_t)e_pos * half + jd];       // position 0 for the rows that do not count
    e_sin = rope.sin_t[(size_t)e_pos * half + jd];
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < rounds; ++it) {
    issue(it + SLOTS - 1, 3);                      // into the slot that was read a round ago
    // Slot `it` has landed: all but the loads issued after its last one.  From round SLOTS - 1 on those are the
    // SLOTS - 1 slots after it; before, the x fragments of the first slots that follow its own and the slots
    // issued in the loop so far.  (Anything else asked for in between only makes this wait for more.)
    if (it >= SLOTS - 1) SG_VMCNT((SLOTS - 1) * L);
    else RingStart<SLOTS, 0>::wait(it);
    sg_u32x4 f[2 * RING_U];
    RingRead<RING_U>::run(at0 + (it % SLOTS) * SLOT_BYTES, f);
#pragma unroll
    for (int u = 0; u < RING_U; ++u)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, f[2 * u]), __builtin_bit_cast(bf16x8, f[2 * u + 1]),
                                                    acc, 0, 0, 0);
  }
  SG_VMCNT(0);                                     // nothing of this wave may still be writing the LDS when it ends

  if (NF && EPI != EPI_ADD) {
    // 1 / sqrt(mean of squares + eps) of every row, summed in a fixed order
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < SSP; ++i) {
      const int t = 4 * (c + 16 * i);
      sum += (t < nf.ss_tiles ? ssp[i].x : 0.f) + (t + 1 < nf.ss_tiles ? ssp[i].y : 0.f) +
             (t + 2 < nf.ss_tiles ? ssp[i].z : 0.f) + (t + 3 < nf.ss_tiles ? ssp[i].w : 0.f);
    }
    if (nf.ss_tiles > 64 * SSP)
      for (int t = 64 * SSP + c; t < nf.ss_tiles; t += 16) sum += nf.ss_in[(size_t)msrc * ss_ld + t];
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    sum += __shfl_xor(sum, 4, 64);
    sum += __shfl_xor(sum, 8, 64);
    if (c == 0) s_rstd[m] = 1.0f / sqrtf(sum * nf.inv_width + nf.eps);
  }

  // sum the waves: acc[i] of lane (col, kb) is weight row 4 kb + i (column of the tile), x row col
#pragma unroll
  for (int i = 0; i < 4; ++i) s_acc[wave][lane * 4 + i] = acc[i];
  __syncthreads();
  float v = 0.f;
  {
    const int src = (((c >> 2) << 4) + m) * 4 + (c & 3);
#pragma unroll
    for (int w = 0; w < SG_WAVES; ++w) v += s_acc[w][src];
  }

  if (EPI == EPI_ADD) {
    const float r = e_old + v;
    if (live) ((float*)outv)[(size_t)m * ldo + n] = r;
    if (NF) {
      const float g = nf.g_f32 ? __uint_as_float(e_g) : __uint_as_float(e_g << 16);
      if (live) nf.x_next[(size_t)m * nf.ldx_next + n] = __float2bfloat16(r * g);
      float q = live ? r * r : 0.f;          // the 16 lanes of a row: sum of squares over this tile's columns
      q += __shfl_xor(q, 1, 64);
      q += __shfl_xor(q, 2, 64);
      q += __shfl_xor(q, 4, 64);
      q += __shfl_xor(q, 8, 64);
      if (c == 0 && m < M) nf.ss_out[(size_t)m * ((gridDim.x + 3) & ~3) + tile] = q;
    }
    return;
  }
  const float rstd = NF ? s_rstd[m] : 1.f;
  const float mine_v = v * rstd;
  float other = 0.f;
  if (EPI == EPI_ROPE || EPI == EPI_SWIGLU) other = __shfl_xor(mine_v, 8, 64);   // the pair's other member
  if (!live) return;
  if (EPI == EPI_ROPE) {
    const int D = rope.D;
    const int head = (int)(n / D), jd = (int)(n - (long)head * D);   // column inside the head
    const int slot = e_slot;
    if (head < rope.Hq + rope.Hkv) {
      // first member (c < 8): x1 cos - x2 sin; second: x2 cos + x1 sin, x1 being the first member's value
      const float o = c < 8 ? mine_v * e_cos - other * e_sin : mine_v * e_cos + other * e_sin;
      if (head < rope.Hq)
        ((bf16*)outv)[(size_t)m * ldo + n] = __float2bfloat16(o);
      else
        rope.k_cache[(((size_t)(slot / rope.page) * rope.Hkv + (head - rope.Hq)) * rope.page + slot % rope.page) * D + jd] =
            __float2bfloat16(o);
    } else {
      rope.v_cache[(((size_t)(slot / rope.page) * rope.Hkv + (head - rope.Hq - rope.Hkv)) * D + jd) * rope.page +
                   slot % rope.page] = __float2bfloat16(mine_v);
    }
  } else if (EPI == EPI_STORE_BF16) {
    ((bf16*)outv)[(size_t)m * ldo + n] = __float2bfloat16(mine_v);
  } else if (EPI == EPI_STORE_F32) {
    ((float*)outv)[(size_t)m * ldo + n] = mine_v;
  } else if (c < 8) {                        // SWIGLU: mine = gate, other = up
    ((bf16*)outv)[(size_t)m * ldo + n] = __float2bfloat16(mine_v / (1.0f + expf(-mine_v)) * other);
  }
}

MIE_EXPORT const char* gemm_bf16_last_error() { return g_mie_error; }
MIE_EXPORT int mie_skinny_max_rows() { return 16; }

// A kernel that wants more LDS than a launch gets by default is told so once per device.
static int allow_lds(const void* kernel, int bytes) {
  static std::mutex lock;
  static std::set<std::pair<int, const void*>> done;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) MIE_FAIL("skinny_gemm: no current device");
  std::lock_guard<std::mutex> g(lock);
  if (done.count({dev, kernel})) return 0;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) MIE_FAIL("skinny_gemm: %d bytes of LDS refused: %s", bytes, hipGetErrorString(e));
  done.insert({dev, kernel});
  return 0;
}

template <bool NF, int SLOTS>
static int launch_epi(int epi, dim3 grid, hipStream_t s, const bf16* X, long ldx, const bf16* W, long ldw, void* out,
                      long ldo, int M, int N, int K, int up_offset, const RopeArgs& rope, const NormArgs& nf) {
  constexpr int lds = SG_WAVES * SLOTS * RING_U * 2 * 1024;
#define SG_LAUNCH(E)                                                                                                    \
  {                                                                                                                     \
    auto kernel = skinny_gemm_kernel<E, NF, SLOTS>;                                                                     \
    if (allow_lds((const void*)kernel, lds)) return -1;                                                                 \
    hipLaunchKernelGGL(kernel, grid, dim3(SG_THREADS), lds, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, nf); \
  }
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

// Slots a wave's ring has.  Four (64 KB a workgroup, two workgroups a compute unit) stream best; three (48 KB,
// three workgroups a compute unit) when that lets all tiles run at once instead of in two rounds.  Chosen from
// the weight's shape alone, never from the batch (the sums do not depend on it anyway).
static int compute_units() {
  static int units[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!units[dev]) {
    int n = 0;
    units[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
  }
  return units[dev];
}
static int slots_for(int tiles) {
  const int cu = compute_units();
  return tiles > 2 * cu && tiles <= 3 * cu ? 3 : 4;
}

static int launch_rows(int tiles, int epi, hipStream_t s, const bf16* X, long ldx, const bf16* W, long ldw, void* out,
                       long ldo, int M, int N, int K, int up_offset, const RopeArgs& rope, const NormArgs* nf) {
  dim3 grid(tiles);
  NormArgs none = {};
  const NormArgs& n = nf ? *nf : none;
  if (slots_for(tiles) == 3)
    return nf ? launch_epi<true, 3>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, n)
              : launch_epi<false, 3>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, n);
  return nf ? launch_epi<true, 4>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, n)
            : launch_epi<false, 4>(epi, grid, s, X, ldx, W, ldw, out, ldo, M, N, K, up_offset, rope, n);
}

static int check_operands(const char* what, const void* X, long ldx, const void* W, long ldw, int M, int K) {
  if (M > 16) MIE_FAIL("%s: %d rows (at most 16)", what, M);
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
