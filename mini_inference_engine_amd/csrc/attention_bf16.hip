// bfloat16 attention on the matrix cores of gfx950, for one head size per build (-DHEAD_DIM=N, a
// multiple of 16 up to 256).  Caches: keys [pages, Hkv, page, D], values [pages, Hkv, D, page].
//
// decode_attention: single-token rows.  One workgroup per (row, kv head, 16 query heads of its group,
// split of the context); its waves take 32-key blocks of the split in turn.  With v_mfma_f32_16x16x32_bf16
//   S^T[key, head]  = K[key, d]  . Q^T[d, head]      A = 16 keys x 32 dims, straight from the key page
//   O^T[d, head]   += V^T[d, key] . P^T[key, head]   A = 16 dims x 32 keys, straight from the value page
// The scores come out with lane % 16 = head and 4 consecutive keys per lane group; that is already
// the layout P^T needs as the B operand of the second product if the 32 keys of its reduction are
// taken in the order (lane group, tile, i), and the value operand is loaded in that same order, so the
// probabilities never leave registers.  Softmax state (max, sum) is one value per lane (its head);
// exponentials are base 2 with scale * log2(e) folded into the scores.  The waves of a workgroup are
// merged through LDS; splits write normalised partials and base-2 log-sum-exps, merged by a second,
// small kernel.  Keys outside [lo, p] get probability 0 by selection and their values are zeroed, so stale
// or poisoned slots never reach the sums.
#include "common.hpp"

#ifndef HEAD_DIM
#error "build with -DHEAD_DIM=<multiple of 16>"
#endif
#if HEAD_DIM % 16 != 0 || HEAD_DIM < 16 || HEAD_DIM > 256
#error "HEAD_DIM must be a multiple of 16 from 16 to 256"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = HEAD_DIM;
constexpr int KS = (D + 31) / 32;      // 32-dim steps of q . k
constexpr int DT = D / 16;             // 16-dim tiles of the output
constexpr int NW = D > 128 ? 2 : 4;    // waves per workgroup (bounded by the LDS the merge needs)
constexpr int BLOCK_KEYS = 32;

union Frag {
  bf16x8 v;
  uint4 q;
  uint2 h[2];
  uint32_t w[4];
};

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

// two floats to two bfloat16 (round to nearest even, one v_cvt_pk_bf16_f32), low half = a
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  const float2_t f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

// max of two numbers neither of which is a NaN, as one instruction (fmaxf adds two more to quiet NaNs)
__device__ __forceinline__ float max_nn(float a, float b) { return __builtin_amdgcn_fmed3f(a, b, INFINITY); }

// max / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one query's or head's lanes), by the lane
// swaps of gfx950 instead of a trip through the LDS: v_permlane16_swap exchanges the odd 16-lane rows of
// its first operand with the even rows of its second, v_permlane32_swap the upper half of the first with
// the lower half of the second; with both operands equal, the pair holds x[l] and x[l ^ 16] (x[l ^ 32]).
__device__ __forceinline__ float quad_max(float x) {      // no NaN among the values
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = max_nn(__uint_as_float(r[0]), __uint_as_float(r[1]));
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return max_nn(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float quad_sum(float x) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// 2^x by the hardware instruction alone: results below 2^-126 are flushed to 0, which a softmax weight may be
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__global__ void __launch_bounds__(NW * 64)
decode_attention_kernel(const bf16* __restrict__ q, long q_stride, const bf16* __restrict__ k_cache,
                        const bf16* __restrict__ v_cache, bf16* __restrict__ out, float* __restrict__ o_part,
                        float* __restrict__ lse_part, const int* __restrict__ block_tables, int max_blocks,
                        const int* __restrict__ positions, int Hq, int Hkv, int head_tiles, int page,
                        float scale_log2, int window, int partition, int num_splits) {
  __shared__ float s_m[NW][16], s_l[NW][16], s_M[16], s_L[16];
  __shared__ float s_o[NW][16][D + 1];
  const int b = blockIdx.x;
  const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y - kvh * head_tiles;
  const int s = blockIdx.z;
  const int G = Hq / Hkv;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int pos = positions[b];
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int begin = (lo & ~(BLOCK_KEYS - 1)) + s * partition;
  const int end = begin + partition < pos + 1 ? begin + partition : pos + 1;
  const int g = ht * 16 + col;
  const bool head_ok = g < G;
  const int head = kvh * G + (head_ok ? g : 0);

  if (begin > pos) {          // this split lies beyond the row's keys (uniform over the workgroup)
    if (num_splits > 1 && threadIdx.x < 16 && ht * 16 + (int)threadIdx.x < G)
      lse_part[((size_t)b * Hq + kvh * G + ht * 16 + threadIdx.x) * num_splits + s] = -INFINITY;
    return;
  }

  const int* bt = block_tables + (size_t)b * max_blocks;
  Frag qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = ks * 32 + kb * 8;
    qf[ks].q = make_uint4(0, 0, 0, 0);
    if (head_ok && d0 < D) qf[ks].q = *reinterpret_cast<const uint4*>(q + (size_t)b * q_stride + (size_t)head * D + d0);
  }

  float m = -INFINITY, l = 0.f;
  f32x4 O[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) O[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int blk = begin + BLOCK_KEYS * wave; blk < end; blk += BLOCK_KEYS * NW) {
    // ---- scores of 32 keys x 16 heads
    f32x4 S[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      S[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      int key = blk + 16 * t + col;
      key = key < pos ? key : pos;                      // never look up pages the row does not have
      const int pg = bt[key / page];
      const bf16* kp = k_cache + (((size_t)pg * Hkv + kvh) * page + key % page) * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d0 = ks * 32 + kb * 8;
        Frag a;
        a.q = make_uint4(0, 0, 0, 0);
        if (d0 < D) a.q = *reinterpret_cast<const uint4*>(kp + d0);
        S[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[ks].v, S[t], 0, 0, 0);
      }
    }
    // ---- values of the same 32 keys, in the order the probabilities sit in registers
    const bool partial = blk + BLOCK_KEYS > pos + 1 || blk < lo;
    Frag va[DT];
    {
      int k0 = blk + 4 * kb, k1 = blk + 16 + 4 * kb;
      const int last = pos & ~3;
      k0 = k0 < last ? k0 : last;
      k1 = k1 < last ? k1 : last;
      const int pg0 = bt[k0 / page], pg1 = bt[k1 / page];
      const bf16* v0 = v_cache + ((size_t)pg0 * Hkv + kvh) * D * page + k0 % page;
      const bf16* v1 = v_cache + ((size_t)pg1 * Hkv + kvh) * D * page + k1 % page;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const size_t drow = (size_t)(dt * 16 + col) * page;
        va[dt].h[0] = *reinterpret_cast<const uint2*>(v0 + drow);
        va[dt].h[1] = *reinterpret_cast<const uint2*>(v1 + drow);
      }
    }
    // ---- online softmax, one head per lane column
    float sv[8];
    bool ok[8];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = blk + 16 * t + 4 * kb + i;
        ok[t * 4 + i] = key >= lo && key <= pos;
        sv[t * 4 + i] = ok[t * 4 + i] ? S[t][i] * scale_log2 : -INFINITY;
        mx = fmaxf(mx, sv[t * 4 + i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);                   // finite: every block taken holds a visible key
    const float alpha = exp2f(m - m_new);
    float p[8], rs = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p[j] = ok[j] ? exp2f(sv[j] - m_new) : 0.f;
      rs += p[j];
    }
    rs += __shfl_xor(rs, 16, 64);
    rs += __shfl_xor(rs, 32, 64);
    l = l * alpha + rs;
    m = m_new;
    Frag pb;
#pragma unroll
    for (int j = 0; j < 4; ++j) pb.w[j] = pack_bf16(p[2 * j], p[2 * j + 1]);
    if (partial) {
      // zero the values of keys outside [lo, pos]: 0 * (stale NaN) must not reach the sum
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t w = va[dt].w[j];
          if (!ok[2 * j]) w &= 0xFFFF0000u;
          if (!ok[2 * j + 1]) w &= 0x0000FFFFu;
          va[dt].w[j] = w;
        }
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      O[dt] *= alpha;
      O[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[dt].v, pb.v, O[dt], 0, 0, 0);
    }
  }

  // ---- merge the waves of the workgroup
  if (kb == 0) {
    s_m[wave][col] = m;
    s_l[wave][col] = l;
  }
  __syncthreads();
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, s_m[w][col]);
  float L = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float mw = s_m[w][col];
    L += mw == -INFINITY ? 0.f : exp2f(mw - M) * s_l[w][col];
  }
  const float f = m == -INFINITY ? 0.f : exp2f(m - M);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) s_o[wave][col][dt * 16 + 4 * kb + i] = O[dt][i] * f;
  if (wave == 0 && kb == 0) {
    s_M[col] = M;
    s_L[col] = L;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 16 * D; e += NW * 64) {
    const int hc = e / D, d = e - hc * D;
    const int gg = ht * 16 + hc;
    if (gg >= G) continue;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += s_o[w][hc][d];
    const float val = sum / s_L[hc];
    const size_t hh = (size_t)b * Hq + kvh * G + gg;
    if (num_splits == 1) {
      out[hh * D + d] = __float2bfloat16(val);
    } else {
      o_part[(hh * num_splits + s) * D + d] = val;
      if (d == 0) lse_part[hh * num_splits + s] = s_M[hc] + log2f(s_L[hc]);
    }
  }
}

// One wave per (row, head): lane s takes the log-sum-exp of split s (the wave reduces max and sum with
// shuffles), then the lanes spread over D and add the splits' partials with all loads of a chunk of 16
// splits issued together: two memory round trips in all, whatever the number of splits.
// (Merging inside the attention kernel by the split that arrives last was tried: the partials have to
// cross the per-XCD L2s, and the device-scope fences that takes cost far more than this launch.)
__global__ void __launch_bounds__(64)
merge_splits_kernel(const float* __restrict__ o_part, const float* __restrict__ lse_part, bf16* __restrict__ out,
                    int num_splits) {
  constexpr int DL = (D + 63) / 64;
  const size_t hh = blockIdx.x;
  const int lane = threadIdx.x;
  const float* lse = lse_part + hh * num_splits;
  const float* op = o_part + hh * num_splits * D;
  float acc[DL];
#pragma unroll
  for (int i = 0; i < DL; ++i) acc[i] = 0.f;
  float W = 0.f;
  float M = -INFINITY;                       // the maximum over all splits first (64 a round)
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const float v = s0 + lane < num_splits ? lse[s0 + lane] : -INFINITY;
    M = fmaxf(M, wave_max(v));
  }
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const float v = s0 + lane < num_splits ? lse[s0 + lane] : -INFINITY;
    const float w = v == -INFINITY ? 0.f : exp2f(v - M);
    W += wave_sum(w);
    const int n = num_splits - s0 < 64 ? num_splits - s0 : 64;
    for (int c = 0; c < n; c += 16) {
      float part[16][DL];
#pragma unroll
      for (int j = 0; j < 16; ++j)
#pragma unroll
        for (int i = 0; i < DL; ++i) {
          const int d = lane + 64 * i;
          part[j][i] = (c + j < n && d < D) ? op[(size_t)(s0 + c + j) * D + d] : 0.f;
        }
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float wj = __shfl(w, (c + j) & 63, 64);
#pragma unroll
        for (int i = 0; i < DL; ++i)
          if (c + j < n && wj != 0.f) acc[i] += wj * part[j][i];    // a split without keys holds no data
      }
    }
  }
  const float inv = 1.0f / W;
#pragma unroll
  for (int i = 0; i < DL; ++i) {
    const int d = lane + 64 * i;
    if (d < D) out[hh * D + d] = __float2bfloat16(acc[i] * inv);
  }
}

// prefill_attention: rows of several tokens, starting anywhere in their request.  The same two
// products as above with "head" replaced by "query": S^T[key, query] = K . Q^T and
// O^T[d, query] += V^T . P^T, so softmax state is again one value per lane (its query).
//
// A workgroup of 4 waves serves one kv head and one stretch of 16 QT queries of a row; its waves own
// PF_NT tiles each (16 queries x 1 head; hpw heads by qpw query tiles), waves_h of them side by side
// over the heads of the group and 4 / waves_h over the queries.  All of them need the same keys: a
// block of 32 keys and values is brought into the LDS once by the whole workgroup (two buffers, the
// next block's loads in flight while the current one is computed, its pages looked up one block
// earlier still), in rows padded so that the fragment reads of the matrix instructions meet no bank
// conflict.  Work per stretch grows with its place in the row (causal), so a workgroup takes stretch
// NS - 1 - i and then stretch i: every workgroup of a row has the same number of blocks to do.
// A block every query of a wave sees whole takes a path without masks; the running maximum m is kept
// in units of scale * log2(e); l is a per-lane partial sum, joined over a query's four lanes at the end.
constexpr int PF_NT = D <= 128 ? 2 : 1;
constexpr int PF_KROW = 2 * D + 16;                 // bytes of a key row in the LDS
constexpr int PF_VROW = 2 * BLOCK_KEYS + 16;        // bytes of a value row (one dim, 32 keys) in the LDS
constexpr int PF_KBYTES = BLOCK_KEYS * PF_KROW;
constexpr int PF_BUF = PF_KBYTES + D * PF_VROW;     // one buffer: keys, then values
constexpr int PF_PIECES = 4 * D;                    // 16-byte pieces of a block's keys (and of its values)
constexpr int PF_PPT = (PF_PIECES + 255) / 256;     // pieces of each a thread carries

__global__ void __launch_bounds__(256)
prefill_attention_kernel(const bf16* __restrict__ q, long q_stride, const bf16* __restrict__ k_cache,
                         const bf16* __restrict__ v_cache, bf16* __restrict__ out,
                         const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ row_start,
                         const int* __restrict__ row_position, int first_row, int Hq, int Hkv, int hpw,
                         int waves_h, int page, float scale_log2, int window) {
  extern __shared__ __align__(16) unsigned char pf_lds[];
  const int row = first_row + blockIdx.y;
  const int G = Hq / Hkv;
  const int qpw = PF_NT / hpw, waves_q = 4 / waves_h, QT = waves_q * qpw;
  const int head_chunks = (G + hpw * waves_h - 1) / (hpw * waves_h);
  const int kvh = blockIdx.z / head_chunks, hc = blockIdx.z - kvh * head_chunks;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int t0 = row_start[row], q_len = row_start[row + 1] - t0, p0 = row_position[row];
  const int NS = (q_len + 16 * QT - 1) / (16 * QT);          // stretches of this row
  if ((int)blockIdx.x >= (NS + 1) / 2) return;               // the whole workgroup, before any barrier
  const int wh = wave % waves_h, wq = wave / waves_h;
  const int* bt = block_tables + (size_t)row * max_blocks;

  for (int pass = 0; pass < 2; ++pass) {
    const int s = pass == 0 ? NS - 1 - (int)blockIdx.x : (int)blockIdx.x;
    if (pass == 1 && s >= NS - 1 - (int)blockIdx.x) break;   // the middle stretch of an odd number has no partner

    // ---- this wave's tiles
    bool tile_ok[PF_NT], q_ok[PF_NT];
    int qpos[PF_NT], qtok[PF_NT], tile_first[PF_NT], tile_last[PF_NT], head[PF_NT];
    Frag qf[PF_NT][KS];
    const int wave_q0 = (s * QT + wq * qpw) * 16;            // first query of the wave
#pragma unroll
    for (int j = 0; j < PF_NT; ++j) {
      const int jh = j % hpw, qt = s * QT + wq * qpw + j / hpw;
      const int g = (hc * waves_h + wh) * hpw + jh;
      tile_ok[j] = g < G && qt * 16 < q_len;
      head[j] = kvh * G + (g < G ? g : 0);
      int qi = qt * 16 + col;
      q_ok[j] = tile_ok[j] && qi < q_len;
      qi = qi < q_len ? qi : q_len - 1;
      qtok[j] = t0 + qi;
      qpos[j] = p0 + qi;
      const int last_q = (qt * 16 + 15 < q_len ? qt * 16 + 15 : q_len - 1);
      tile_first[j] = p0 + qt * 16;
      tile_last[j] = p0 + last_q;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d0 = ks * 32 + kb * 8;
        qf[j][ks].q = make_uint4(0, 0, 0, 0);
        if (tile_ok[j] && d0 < D)
          qf[j][ks].q = *reinterpret_cast<const uint4*>(q + (size_t)qtok[j] * q_stride + (size_t)head[j] * D + d0);
      }
    }
    // keys the wave's queries can see, and the workgroup's (the union over its waves)
    int wave_last = (wave_q0 + qpw * 16 < q_len ? wave_q0 + qpw * 16 : q_len) - 1;
    const int wave_kmax = wave_q0 < q_len ? p0 + wave_last : -1;       // -1: the wave has no query
    const int wave_kmin = window > 0 ? p0 + wave_q0 - window + 1 : 0;
    const int end_q = (s + 1) * QT * 16 < q_len ? (s + 1) * QT * 16 : q_len;
    const int kmax = p0 + end_q - 1;
    int kmin = window > 0 ? p0 + s * QT * 16 - window + 1 : 0;
    kmin = kmin > 0 ? kmin : 0;
    const int blk0 = kmin & ~(BLOCK_KEYS - 1);
    const int last_blk = kmax & ~(BLOCK_KEYS - 1);

    float m[PF_NT], l[PF_NT];
    f32x4 O[PF_NT][DT];
#pragma unroll
    for (int j = 0; j < PF_NT; ++j) {
      m[j] = -INFINITY;
      l[j] = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) O[j][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- bringing a block into the LDS: piece c of the keys is 8 dims of one key, piece c of the values
    // 8 keys of one dim.  Where the pieces lie (page and place in it) is found by walking the block table:
    // [walk_start, walk_start + page) is the page of the block looked up last, and a key at most 31 past
    // a block's start lies at most two pages on.  Addresses are clamped to the row's own keys.
    struct Where {
      int kpg[PF_PPT], koff[PF_PPT], vpg[PF_PPT], voff[PF_PPT];
    };
    struct Pieces {
      uint4 k[PF_PPT], v[PF_PPT];
    };
    int walk_idx = blk0 / page, walk_start = walk_idx * page;
    auto lookup = [&](Where& Wh, int blk) {
      blk = blk < last_blk ? blk : last_blk;           // beyond the last block: the last one again
      while (blk >= walk_start + page) {
        walk_start += page;
        ++walk_idx;
      }
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + 256 * i < PF_PIECES ? tid + 256 * i : 0;
        int key = blk + c / (D / 8);
        key = key < kmax ? key : kmax;
        int rel = key - walk_start;
        int w = (rel >= page ? 1 : 0) + (rel >= 2 * page ? 1 : 0);
        Wh.kpg[i] = bt[walk_idx + w];
        Wh.koff[i] = rel - w * page;
        key = blk + (c & 3) * 8;
        key = key < (kmax & ~7) ? key : (kmax & ~7);
        rel = key - walk_start;
        w = (rel >= page ? 1 : 0) + (rel >= 2 * page ? 1 : 0);
        Wh.vpg[i] = bt[walk_idx + w];
        Wh.voff[i] = rel - w * page;
      }
    };
    auto fetch = [&](Pieces& P, const Where& Wh) {
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + 256 * i < PF_PIECES ? tid + 256 * i : 0;
        P.k[i] = *reinterpret_cast<const uint4*>(
            k_cache + (((size_t)Wh.kpg[i] * Hkv + kvh) * page + Wh.koff[i]) * D + (c % (D / 8)) * 8);
        P.v[i] = *reinterpret_cast<const uint4*>(
            v_cache + (((size_t)Wh.vpg[i] * Hkv + kvh) * D + (c >> 2)) * page + Wh.voff[i]);
      }
    };
    auto stash = [&](Pieces& P, int buf, int blk) {
      unsigned char* base = pf_lds + buf * PF_BUF;
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + 256 * i;
        if (c >= PF_PIECES) continue;
        *reinterpret_cast<uint4*>(base + (c / (D / 8)) * PF_KROW + (c % (D / 8)) * 16) = P.k[i];
        uint4 v = P.v[i];
        const int key0 = blk + (c & 3) * 8;
        if (key0 + 7 > kmax) {
          // slots after the row's last key may be stale: zero them (0 * NaN must not reach the sum)
          uint32_t* w = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (key0 + 2 * e > kmax) w[e] &= 0xFFFF0000u;
            if (key0 + 2 * e + 1 > kmax) w[e] &= 0x0000FFFFu;
          }
        }
        *reinterpret_cast<uint4*>(base + PF_KBYTES + (c >> 2) * PF_VROW + (c & 3) * 16) = v;
      }
    };

    // ---- one block for all tiles of the wave, stage by stage (scores of every tile, softmax of every
    // tile, outputs of every tile), so that the matrix and the vector unit have independent work side by side
    auto compute = [&](int buf, int blk) {
      const unsigned char* Kb = pf_lds + buf * PF_BUF;
      const unsigned char* Vb = Kb + PF_KBYTES;
      Frag a[2][KS], va[DT];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int d0 = ks * 32 + kb * 8;
          a[t][ks].q = make_uint4(0, 0, 0, 0);
          if (d0 < D) a[t][ks].q = *reinterpret_cast<const uint4*>(Kb + (16 * t + col) * PF_KROW + d0 * 2);
        }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const unsigned char* vr = Vb + (dt * 16 + col) * PF_VROW + 8 * kb;
        va[dt].h[0] = *reinterpret_cast<const uint2*>(vr);
        va[dt].h[1] = *reinterpret_cast<const uint2*>(vr + 32);
      }
      f32x4 S[PF_NT][2];
      bool whole = true;      // every query of every tile sees every key of the block (uniform over the wave)
#pragma unroll
      for (int j = 0; j < PF_NT; ++j) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          S[j][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            S[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][ks].v, qf[j][ks].v, S[j][t], 0, 0, 0);
        }
        whole = whole && (!tile_ok[j] || (blk + BLOCK_KEYS - 1 <= tile_first[j] &&
                                          (window <= 0 || blk >= tile_last[j] - window + 1)));
      }
      float p[PF_NT][8], alpha[PF_NT];
      if (whole) {
#pragma unroll
        for (int j = 0; j < PF_NT; ++j) {
          float mx = max_nn(max_nn(max_nn(S[j][0][0], S[j][0][1]), max_nn(S[j][0][2], S[j][0][3])),
                            max_nn(max_nn(S[j][1][0], S[j][1][1]), max_nn(S[j][1][2], S[j][1][3])));
          mx = quad_max(mx);
          const float m_new = max_nn(m[j], mx * scale_log2);
          alpha[j] = fast_exp2(m[j] - m_new);
          m[j] = m_new;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) p[j][t * 4 + i] = fast_exp2(fmaf(S[j][t][i], scale_log2, -m_new));
        }
      } else {
#pragma unroll
        for (int j = 0; j < PF_NT; ++j) {
          const int hi = tile_ok[j] ? qpos[j] : -1;            // a tile that does not exist sees nothing
          const int lo = window > 0 ? hi - window + 1 : 0;
          bool ok[8];
          float mx = -INFINITY;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int key = blk + 16 * t + 4 * kb + i;
              ok[t * 4 + i] = key >= lo && key <= hi;
              mx = max_nn(mx, ok[t * 4 + i] ? S[j][t][i] : -INFINITY);
            }
          mx = quad_max(mx);
          const float m_new = max_nn(m[j], mx * scale_log2);
          // a query may see none of this block's keys (it lies before the block, or the block before its window)
          alpha[j] = m_new == -INFINITY ? 1.f : fast_exp2(m[j] - m_new);
          m[j] = m_new;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              p[j][t * 4 + i] = ok[t * 4 + i] ? fast_exp2(fmaf(S[j][t][i], scale_log2, -m_new)) : 0.f;
        }
      }
      Frag pb[PF_NT];
      bool moved = false;
#pragma unroll
      for (int j = 0; j < PF_NT; ++j) {
        const float rs = ((p[j][0] + p[j][1]) + (p[j][2] + p[j][3])) + ((p[j][4] + p[j][5]) + (p[j][6] + p[j][7]));
        l[j] = l[j] * alpha[j] + rs;
#pragma unroll
        for (int e = 0; e < 4; ++e) pb[j].w[e] = pack_bf16(p[j][2 * e], p[j][2 * e + 1]);
        moved = moved || alpha[j] != 1.f;
      }
      if (__builtin_amdgcn_ballot_w64(moved) != 0) {          // the maxima rarely move after the first blocks
#pragma unroll
        for (int j = 0; j < PF_NT; ++j)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) O[j][dt] *= alpha[j];
      }
#pragma unroll
      for (int j = 0; j < PF_NT; ++j)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          O[j][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[dt].v, pb[j].v, O[j][dt], 0, 0, 0);
    };

    // ---- the blocks, two buffers: block i is computed while block i + 1 travels and the pages of block
    // i + 2 are looked up; one barrier a block
    Where wh_next;
    Pieces pc;
    lookup(wh_next, blk0);
    fetch(pc, wh_next);
    lookup(wh_next, blk0 + BLOCK_KEYS);
    __syncthreads();                                   // the previous stretch is done with the buffers
    stash(pc, 0, blk0);
    __syncthreads();
    int buf = 0;
    for (int blk = blk0; blk <= kmax; blk += BLOCK_KEYS, buf ^= 1) {
      const bool more = blk + BLOCK_KEYS <= kmax;      // uniform over the workgroup
      if (more) {
        fetch(pc, wh_next);
        lookup(wh_next, blk + 2 * BLOCK_KEYS);
      }
      if (blk <= wave_kmax && blk + BLOCK_KEYS > wave_kmin) compute(buf, blk);
      if (more) stash(pc, buf ^ 1, blk + BLOCK_KEYS);
      __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < PF_NT; ++j) {
      const float total = quad_sum(l[j]);
      if (!q_ok[j]) continue;
      const float inv = 1.0f / total;
      bf16* op = out + ((size_t)qtok[j] * Hq + head[j]) * D + 4 * kb;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        uint2 st;
        st.x = pack_bf16(O[j][dt][0] * inv, O[j][dt][1] * inv);
        st.y = pack_bf16(O[j][dt][2] * inv, O[j][dt][3] * inv);
        *reinterpret_cast<uint2*>(op + dt * 16) = st;
      }
    }
  }
}

MIE_EXPORT const char* attention_bf16_last_error() { return g_mie_error; }
MIE_EXPORT int mie_attention_bf16_head_dim() { return D; }
MIE_EXPORT int mie_decode_block_keys() { return BLOCK_KEYS * NW; }

// q: token b is row b (single-token rows lead the flattened batch).  partition: keys per split, a
// multiple of mie_decode_block_keys().  o_part [rows, Hq, splits, D] and lse_part [rows, Hq, splits]
// float are needed when num_splits > 1.
MIE_EXPORT int mie_decode_attention(const void* q, long q_stride, const void* k_cache, const void* v_cache, void* out,
                                    float* o_part, float* lse_part, const int* block_tables, int max_blocks,
                                    const int* positions, int rows, int Hq, int Hkv, int head_dim, int page,
                                    float scale, int window, int partition, int num_splits, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (head_dim != D) MIE_FAIL("decode_attention: built for head_dim %d, called with %d", D, head_dim);
  if (Hkv <= 0 || Hq % Hkv) MIE_FAIL("decode_attention: %d query heads on %d kv heads", Hq, Hkv);
  if (page < 16 || page % 16) MIE_FAIL("decode_attention: page size %d (multiples of 16)", page);
  if (partition <= 0 || partition % (BLOCK_KEYS * NW)) MIE_FAIL("decode_attention: partition %d is no multiple of %d", partition, BLOCK_KEYS * NW);
  if (num_splits < 1 || num_splits > 65535) MIE_FAIL("decode_attention: %d splits", num_splits);
  if (num_splits > 1 && (!o_part || !lse_part)) MIE_FAIL("decode_attention: splits need partial buffers");
  if (q_stride < (long)Hq * D || (q_stride % 8) || ((uintptr_t)q % 16)) MIE_FAIL("decode_attention: q stride %ld / alignment", q_stride);
  if (max_blocks <= 0) MIE_FAIL("decode_attention: max_blocks %d", max_blocks);
  const int G = Hq / Hkv, head_tiles = (G + 15) / 16;
  if ((long)Hkv * head_tiles > 65535) MIE_FAIL("decode_attention: too many head tiles for the grid");
  dim3 grid(rows, Hkv * head_tiles, num_splits), block(NW * 64);
  hipLaunchKernelGGL(decode_attention_kernel, grid, block, 0, stream, (const bf16*)q, q_stride, (const bf16*)k_cache,
                     (const bf16*)v_cache, (bf16*)out, o_part, lse_part, block_tables, max_blocks, positions, Hq, Hkv,
                     head_tiles, page, scale * 1.4426950408889634f, window, partition, num_splits);
  MIE_CHECK_LAUNCH("decode_attention");
  if (num_splits > 1) {
    hipLaunchKernelGGL(merge_splits_kernel, dim3(rows * Hq), dim3(64), 0, stream, o_part, lse_part, (bf16*)out, num_splits);
    MIE_CHECK_LAUNCH("merge_splits");
  }
  return 0;
}

// Rows first_row .. first_row + rows - 1 of the step (those of more than one token).  q and out are
// indexed by flat token; row_start [all rows + 1], row_position [all rows] as the step gives them.
MIE_EXPORT int mie_prefill_attention(const void* q, long q_stride, const void* k_cache, const void* v_cache, void* out,
                                     const int* block_tables, int max_blocks, const int* row_start,
                                     const int* row_position, int first_row, int rows, int max_row_tokens, int Hq,
                                     int Hkv, int head_dim, int page, float scale, int window, hipStream_t stream) {
  if (rows <= 0 || max_row_tokens <= 0) return 0;
  if (head_dim != D) MIE_FAIL("prefill_attention: built for head_dim %d, called with %d", D, head_dim);
  if (Hkv <= 0 || Hq % Hkv) MIE_FAIL("prefill_attention: %d query heads on %d kv heads", Hq, Hkv);
  if (page < 16 || page % 16) MIE_FAIL("prefill_attention: page size %d (multiples of 16)", page);
  if (q_stride < (long)Hq * D || (q_stride % 8) || ((uintptr_t)q % 16) || ((uintptr_t)out % 8))
    MIE_FAIL("prefill_attention: q stride %ld / alignment", q_stride);
  if (max_blocks <= 0) MIE_FAIL("prefill_attention: max_blocks %d", max_blocks);
  const int G = Hq / Hkv;
  int hpw = PF_NT;                       // heads of a kv group per wave: the largest power of two <= min(G, PF_NT)
  while (hpw > G) hpw >>= 1;
  const int head_waves = (G + hpw - 1) / hpw;
  const int waves_h = head_waves >= 3 ? 4 : head_waves;       // waves side by side over the heads: 1, 2 or 4
  const int head_chunks = (G + hpw * waves_h - 1) / (hpw * waves_h);
  const int stretch = (4 / waves_h) * (PF_NT / hpw) * 16;      // queries a workgroup serves at a time
  const long stretches = (max_row_tokens + stretch - 1) / stretch;
  const long gx = (stretches + 1) / 2;                        // a workgroup takes a late stretch and an early one
  if (rows > 65535 || (long)Hkv * head_chunks > 65535) MIE_FAIL("prefill_attention: grid too large (%d rows)", rows);
  constexpr int lds_bytes = 2 * PF_BUF;
  static bool lds_allowed[64] = {};
  if (lds_bytes > 64 * 1024) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) MIE_FAIL("prefill_attention: no current device");
    if (!lds_allowed[dev]) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_attention_kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) MIE_FAIL("prefill_attention: %d bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
      lds_allowed[dev] = true;
    }
  }
  dim3 grid((unsigned)gx, rows, Hkv * head_chunks), block(256);
  hipLaunchKernelGGL(prefill_attention_kernel, grid, block, lds_bytes, stream, (const bf16*)q, q_stride,
                     (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, block_tables, max_blocks, row_start,
                     row_position, first_row, Hq, Hkv, hpw, waves_h, page, scale * 1.4426950408889634f, window);
  MIE_CHECK_LAUNCH("prefill_attention");
  return 0;
}
