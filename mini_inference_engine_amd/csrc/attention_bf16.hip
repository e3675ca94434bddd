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
#include "attention_bf16_common.hpp"

constexpr int NW_SPLIT = D > 128 ? 2 : 4;    // waves per workgroup (bounded by the LDS the merge of the waves needs)
// When rows and heads alone fill the GPU the context is not split and there is no second kernel; a workgroup then
// has a whole context to read, and eight waves keep twice the loads in flight for it: as long as there are
// fewer than two workgroups a compute unit.  With more, the compute units are kept busy by the number of
// workgroups, and four waves each are faster (256 rows x 4 kv heads of 512 keys: 24.8 against 32.9 us; 64 rows of
// 2,048 keys: 27.8 against 24.1).
constexpr int NW_WHOLE = D > 128 ? 2 : (D > 64 ? 4 : 8);
constexpr long NW_WHOLE_BELOW = 512;         // workgroups from which on a workgroup is NW_SPLIT waves again

// What the kernel needs to finish the q/k/v projection of its row itself (FROM_SUMS): the projection's
// float32 sums, split over K or not, instead of q; the angle tables; where the row's new key and value go.
// A workgroup then owns everything of its (row, kv head): it adds the splits up, rotates its group's q heads
// (kept in the LDS) and its k head, writes k and v to their cache slot, and goes on as if another kernel had.
// Only for unsplit contexts and groups of up to 16 heads (one workgroup per row and kv head).
struct ProjectionSums {
  const float* part;         // [splits, rows, ld]: q heads, k heads, v heads
  int splits;
  size_t split_stride;       // floats from one split to the next
  long ld;
  const float* cos_t;        // [positions, D / 2]
  const float* sin_t;
  const int* slots;          // [rows] cache slot of each row's token
};

template <int NW, bool FROM_SUMS>
__global__ void __launch_bounds__(NW * 64)
decode_attention_kernel(const bf16* __restrict__ q, long q_stride, bf16* k_cache, bf16* v_cache,
                        bf16* __restrict__ out, float* __restrict__ o_part,
                        float* __restrict__ lse_part, const int* __restrict__ block_tables, int max_blocks,
                        const int* __restrict__ positions, int Hq, int Hkv, int head_tiles, int page,
                        float scale_log2, int window, int partition, int num_splits, ProjectionSums proj) {
  __shared__ float s_m[NW][16], s_l[NW][16], s_M[16], s_L[16];
  __shared__ float s_o[NW][16][D + 1];
  __shared__ __align__(16) bf16 s_q[FROM_SUMS ? 16 : 1][D];
  __shared__ __align__(16) bf16 s_k[FROM_SUMS ? D : 1], s_v[FROM_SUMS ? D : 1];   // the row's own new key and value
  const int b = blockIdx.x;
  const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y - kvh * head_tiles;
  const int s = blockIdx.z;
  const int G = Hq / Hkv;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int g = ht * 16 + col;
  const bool head_ok = g < G;
  const int head = kvh * G + (head_ok ? g : 0);
  const int* bt = block_tables + (size_t)b * max_blocks;

  // Everything that can be asked for before the row's length is known is asked for first: the queries
  // and, without a window, the first block of keys and values (pages are looked up by key index alone,
  // clamped to the table; entries past the row's pages name the scratch page, whose contents are masked).
  Frag qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = ks * 32 + kb * 8;
    qf[ks].q = make_uint4(0, 0, 0, 0);
    if (!FROM_SUMS && head_ok && d0 < D) qf[ks].q = *reinterpret_cast<const uint4*>(q + (size_t)b * q_stride + (size_t)head * D + d0);
  }
  struct KeyBlock {
    Frag a[2][KS];      // keys: 16 keys x 32 dims each
    Frag va[DT];        // values: 16 dims x 32 keys each, in the order the probabilities sit in registers
  };
  const int last_page = max_blocks - 1;
  auto load_block = [&](KeyBlock& B, int blk) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = blk + 16 * t + col;
      int pi = key / page;
      pi = pi < last_page ? pi : last_page;
      const bf16* kp = k_cache + (((size_t)bt[pi] * Hkv + kvh) * page + key % page) * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d0 = ks * 32 + kb * 8;
        B.a[t][ks].q = *reinterpret_cast<const uint4*>(kp + (d0 < D ? d0 : 0));
      }
    }
    const int k0 = blk + 4 * kb, k1 = blk + 16 + 4 * kb;
    int p0 = k0 / page, p1 = k1 / page;
    p0 = p0 < last_page ? p0 : last_page;
    p1 = p1 < last_page ? p1 : last_page;
    const bf16* v0 = v_cache + ((size_t)bt[p0] * Hkv + kvh) * D * page + k0 % page;
    const bf16* v1 = v_cache + ((size_t)bt[p1] * Hkv + kvh) * D * page + k1 % page;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const size_t drow = (size_t)(dt * 16 + col) * page;
      B.va[dt].h[0] = *reinterpret_cast<const uint2*>(v0 + drow);
      B.va[dt].h[1] = *reinterpret_cast<const uint2*>(v1 + drow);
    }
  };
  constexpr bool AHEAD = D <= 128;          // two blocks in registers; larger heads have no room for it
  KeyBlock b0, b1;
  const int pos_raw = positions[b];
  int begin0 = s * partition;               // the split's first key when there is no window
  if (AHEAD && window <= 0) load_block(b0, begin0 + BLOCK_KEYS * wave);

  const int pos = pos_raw;
  if (FROM_SUMS) {
    // the row's own q, k and v from the projection's sums (the expressions of the kernel that does this alone)
    const int slot = proj.slots[b], half = D >> 1;
    const float* pr = proj.part + (size_t)b * proj.ld;
    const float* cr = proj.cos_t + (size_t)pos * half;
    const float* sr = proj.sin_t + (size_t)pos * half;
    bf16* kdst = k_cache + (((size_t)(slot / page) * Hkv + kvh) * page + (size_t)(slot % page)) * D;
    for (int t = threadIdx.x; t < (G + 1) * half; t += NW * 64) {
      const int hh = t / half, j = t - hh * half;
      const float* src = pr + (size_t)(hh < G ? kvh * G + hh : Hq + kvh) * D + j;
      float x1 = 0.f, x2 = 0.f;
      add_splits(x1, src, proj.splits, proj.split_stride);
      add_splits(x2, src + half, proj.splits, proj.split_stride);
      const float c = cr[j], sn = sr[j];
      float o1, o2;
      rotate_pair(x1, x2, c, sn, o1, o2);
      bf16* dst = hh < G ? s_q[hh] : s_k;
      dst[j] = __float2bfloat16(o1);
      dst[j + half] = __float2bfloat16(o2);
      if (hh == G) {
        kdst[j] = __float2bfloat16(o1);
        kdst[j + half] = __float2bfloat16(o2);
      }
    }
    bf16* vdst = v_cache + ((size_t)(slot / page) * Hkv + kvh) * page * D + (size_t)(slot % page);
    for (int d = threadIdx.x; d < D; d += NW * 64) {
      float v = 0.f;
      add_splits(v, pr + (size_t)(Hq + Hkv + kvh) * D + d, proj.splits, proj.split_stride);
      vdst[(size_t)d * page] = __float2bfloat16(v);
      s_v[d] = __float2bfloat16(v);
    }
    // The waves meet over what went into the LDS only; the stores to the cache are not waited for, because
    // nobody here reads them back: the block that holds the row's own key takes it from the LDS (compute()).
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + kb * 8;
      if (head_ok && d0 < D) qf[ks].q = *reinterpret_cast<const uint4*>(&s_q[g][d0]);
    }
  }
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int begin = (lo & ~(BLOCK_KEYS - 1)) + s * partition;
  const int end = begin + partition < pos + 1 ? begin + partition : pos + 1;

  if (begin > pos) {          // this split lies beyond the row's keys (uniform over the workgroup)
    if (num_splits > 1 && threadIdx.x < 16 && ht * 16 + (int)threadIdx.x < G)
      lse_part[((size_t)b * Hq + kvh * G + ht * 16 + threadIdx.x) * num_splits + s] = -INFINITY;
    return;
  }

  float m = -INFINITY, l = 0.f;
  f32x4 O[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) O[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](KeyBlock& B, int blk) {
    if (FROM_SUMS && pos >= blk && pos < blk + BLOCK_KEYS) {       // (the same for the whole wave)
      // what was loaded for the row's own key is whatever its slot held: the key and value come from the LDS
#pragma unroll
      for (int t = 0; t < 2; ++t)
        if (blk + 16 * t + col == pos) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 32 + kb * 8;
            B.a[t][ks].q = *reinterpret_cast<const uint4*>(&s_k[d0 < D ? d0 : 0]);
          }
        }
#pragma unroll
      for (int wi = 0; wi < 4; ++wi) {                           // word wi of a value fragment: two keys
        const int key = blk + 16 * (wi >> 1) + 4 * kb + 2 * (wi & 1);
        const bool low = key == pos, high = key + 1 == pos;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const uint32_t nv = (uint32_t)__bfloat16_as_ushort(s_v[dt * 16 + col]);
          const uint32_t w = B.va[dt].w[wi];
          B.va[dt].w[wi] = low ? (w & 0xFFFF0000u) | nv : (high ? (w & 0x0000FFFFu) | (nv << 16) : w);
        }
      }
    }
    if (D % 32 != 0) {
      // the last 32-dim step of the keys is half empty: its upper lanes were loaded from dim 0
#pragma unroll
      for (int t = 0; t < 2; ++t)
        if ((KS - 1) * 32 + kb * 8 >= D) B.a[t][KS - 1].q = make_uint4(0, 0, 0, 0);
    }
    // ---- scores of 32 keys x 16 heads
    f32x4 S[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      S[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        S[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(B.a[t][ks].v, qf[ks].v, S[t], 0, 0, 0);
    }
    const bool partial = blk + BLOCK_KEYS > pos + 1 || blk < lo;
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
          uint32_t w = B.va[dt].w[j];
          if (!ok[2 * j]) w &= 0xFFFF0000u;
          if (!ok[2 * j + 1]) w &= 0x0000FFFFu;
          B.va[dt].w[j] = w;
        }
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      O[dt] *= alpha;
      O[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(B.va[dt].v, pb.v, O[dt], 0, 0, 0);
    }
  };

  constexpr int STEP = BLOCK_KEYS * NW;     // keys from one block of a wave to its next
  const int first = begin + BLOCK_KEYS * wave;
  if (AHEAD) {
    if (window > 0) load_block(b0, first);  // with a window the split's start had to wait for the row's length
    const int part_end = begin + partition;   // nothing is asked for beyond the split's own keys
    for (int blk = first; blk < end; blk += 2 * STEP) {
      if (blk + STEP < part_end) load_block(b1, blk + STEP);           // in flight while block 0 is computed
      compute(b0, blk);
      if (blk + 2 * STEP < part_end) load_block(b0, blk + 2 * STEP);
      if (blk + STEP < end) compute(b1, blk + STEP);
    }
  } else {
    for (int blk = first; blk < end; blk += STEP) {
      load_block(b0, blk);
      compute(b0, blk);
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
  // Sixteen splits' partial outputs at a time.  The first sixteen are asked for before their weights are
  // known, so that the kernel waits for memory once and not twice; every load is unconditional, from an
  // address clamped into the operand (what is read for a split or a dim that does not exist is not used).
  float part[16][DL];
  auto ask = [&](int first) {
#pragma unroll
    for (int j = 0; j < 16; ++j)
#pragma unroll
      for (int i = 0; i < DL; ++i) {
        const int d = lane + 64 * i, sp = first + j;
        part[j][i] = op[(size_t)(sp < num_splits ? sp : num_splits - 1) * D + (d < D ? d : 0)];
      }
  };
  ask(0);
  float W = 0.f;
  float M = -INFINITY;                       // the maximum over all splits first (64 a round)
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const float v = lse[s0 + lane < num_splits ? s0 + lane : 0];
    M = fmaxf(M, wave_max(s0 + lane < num_splits ? v : -INFINITY));
  }
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const float vv = lse[s0 + lane < num_splits ? s0 + lane : 0];
    const float v = s0 + lane < num_splits ? vv : -INFINITY;
    const float w = v == -INFINITY ? 0.f : exp2f(v - M);
    W += wave_sum(w);
    const int n = num_splits - s0 < 64 ? num_splits - s0 : 64;
    for (int c = 0; c < n; c += 16) {
      if (s0 + c > 0) ask(s0 + c);
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float wj = __shfl(w, (c + j) & 63, 64);
#pragma unroll
        for (int i = 0; i < DL; ++i)
          if (c + j < n && wj != 0.f && lane + 64 * i < D) acc[i] += wj * part[j][i];    // a split without keys holds no data
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

MIE_EXPORT const char* attention_bf16_last_error() { return g_mie_error; }
MIE_EXPORT int mie_attention_bf16_head_dim() { return D; }
MIE_EXPORT int mie_decode_block_keys() { return BLOCK_KEYS * NW_SPLIT; }

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
  if (partition <= 0 || partition % (BLOCK_KEYS * NW_SPLIT)) MIE_FAIL("decode_attention: partition %d is no multiple of %d", partition, BLOCK_KEYS * NW_SPLIT);
  if (num_splits < 1 || num_splits > 65535) MIE_FAIL("decode_attention: %d splits", num_splits);
  if (num_splits > 1 && (!o_part || !lse_part)) MIE_FAIL("decode_attention: splits need partial buffers");
  if (q_stride < (long)Hq * D || (q_stride % 8) || ((uintptr_t)q % 16)) MIE_FAIL("decode_attention: q stride %ld / alignment", q_stride);
  if (max_blocks <= 0) MIE_FAIL("decode_attention: max_blocks %d", max_blocks);
  const int G = Hq / Hkv, head_tiles = (G + 15) / 16;
  if ((long)Hkv * head_tiles > 65535) MIE_FAIL("decode_attention: too many head tiles for the grid");
  dim3 grid(rows, Hkv * head_tiles, num_splits);
  // (the kernel writes the caches only when it is given the projection's sums)
  bf16* kc = (bf16*)const_cast<void*>(k_cache);
  bf16* vc = (bf16*)const_cast<void*>(v_cache);
  if (num_splits == 1 && NW_WHOLE != NW_SPLIT && (long)rows * Hkv * head_tiles < NW_WHOLE_BELOW)
    hipLaunchKernelGGL((decode_attention_kernel<NW_WHOLE, false>), grid, dim3(NW_WHOLE * 64), 0, stream, (const bf16*)q, q_stride,
                       kc, vc, (bf16*)out, o_part, lse_part, block_tables, max_blocks, positions, Hq, Hkv, head_tiles, page,
                       scale * 1.4426950408889634f, window, partition, num_splits, ProjectionSums{});
  else
    hipLaunchKernelGGL((decode_attention_kernel<NW_SPLIT, false>), grid, dim3(NW_SPLIT * 64), 0, stream, (const bf16*)q, q_stride,
                       kc, vc, (bf16*)out, o_part, lse_part, block_tables, max_blocks, positions, Hq, Hkv, head_tiles, page,
                       scale * 1.4426950408889634f, window, partition, num_splits, ProjectionSums{});
  MIE_CHECK_LAUNCH("decode_attention");
  if (num_splits > 1) {
    hipLaunchKernelGGL(merge_splits_kernel, dim3(rows * Hq), dim3(64), 0, stream, o_part, lse_part, (bf16*)out, num_splits);
    MIE_CHECK_LAUNCH("merge_splits");
  }
  return 0;
}


// The q/k/v projection's end and the attention in one kernel, for steps whose rows and kv heads alone fill
// the GPU (contexts unsplit).  part [splits, rows, ld] float32: the projection's sums (q heads, k heads, v
// heads), to be added up in split order; rotary over the whole head with angles from cos / sin [positions,
// D / 2]; the row's k and v go to cache slot slots[row], which must be the slot of key positions[row] in the
// row's block table.  Groups of up to 16 query heads a kv head.  partition as for mie_decode_attention (at least the
// longest context).
MIE_EXPORT int mie_decode_attention_from_sums(const float* part, int splits, long split_stride, long ld, const float* cos_t,
                                              const float* sin_t, const int* slots, void* k_cache, void* v_cache, void* out,
                                              const int* block_tables, int max_blocks, const int* positions, int rows, int Hq,
                                              int Hkv, int head_dim, int page, float scale, int window, int partition,
                                              hipStream_t stream) {
  if (rows <= 0) return 0;
  if (head_dim != D) MIE_FAIL("decode_attention_from_sums: built for head_dim %d, called with %d", D, head_dim);
  if (Hkv <= 0 || Hq % Hkv) MIE_FAIL("decode_attention_from_sums: %d query heads on %d kv heads", Hq, Hkv);
  if (Hq / Hkv > 16) MIE_FAIL("decode_attention_from_sums: groups of %d query heads (at most 16)", Hq / Hkv);
  if (page < 16 || page % 16) MIE_FAIL("decode_attention_from_sums: page size %d (multiples of 16)", page);
  if (partition <= 0 || partition % (BLOCK_KEYS * NW_SPLIT)) MIE_FAIL("decode_attention_from_sums: partition %d is no multiple of %d", partition, BLOCK_KEYS * NW_SPLIT);
  if (!part || !cos_t || !sin_t || !slots || !k_cache || !v_cache || !out || !positions || !block_tables) MIE_FAIL("decode_attention_from_sums: null operand");
  if (splits < 1 || ld < (long)(Hq + 2 * Hkv) * D || (splits > 1 && split_stride < (long)rows * ld)) MIE_FAIL("decode_attention_from_sums: %d splits, stride %ld, row stride %ld", splits, split_stride, ld);
  if (max_blocks <= 0 || Hkv > 65535) MIE_FAIL("decode_attention_from_sums: max_blocks %d, %d kv heads", max_blocks, Hkv);
  const ProjectionSums proj = {part, splits, (size_t)split_stride, ld, cos_t, sin_t, slots};
  dim3 grid(rows, Hkv, 1);
  if ((long)rows * Hkv < NW_WHOLE_BELOW)
    hipLaunchKernelGGL((decode_attention_kernel<NW_WHOLE, true>), grid, dim3(NW_WHOLE * 64), 0, stream, (const bf16*)nullptr, 0L,
                       (bf16*)k_cache, (bf16*)v_cache, (bf16*)out, (float*)nullptr, (float*)nullptr, block_tables, max_blocks,
                       positions, Hq, Hkv, 1, page, scale * 1.4426950408889634f, window, partition, 1, proj);
  else
    hipLaunchKernelGGL((decode_attention_kernel<NW_SPLIT, true>), grid, dim3(NW_SPLIT * 64), 0, stream, (const bf16*)nullptr, 0L,
                       (bf16*)k_cache, (bf16*)v_cache, (bf16*)out, (float*)nullptr, (float*)nullptr, block_tables, max_blocks,
                       positions, Hq, Hkv, 1, page, scale * 1.4426950408889634f, window, partition, 1, proj);
  MIE_CHECK_LAUNCH("decode_attention_from_sums");
  return 0;
}


// ---- the same for callers that cannot allocate (decode_attention_static.hpp)
#include "decode_attention_static.hpp"
#include <mutex>

// Partial results of a split context: the library's own device memory, one copy on every GPU.
// In host code this name is only a stand-in for the symbol; the device address comes from
// hipGetSymbolAddress, per device, and only that address is ever handed to a kernel.
static __device__ __align__(256) float scratch[MIE_DECODE_STATIC_SCRATCH_BYTES / sizeof(float)];

constexpr int MAX_DEVICES = 64;
static float* g_scratch_of_device[MAX_DEVICES];
static std::mutex g_scratch_lock;

static int scratch_for_current_device(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) MIE_FAIL("decode_attention_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= MAX_DEVICES) MIE_FAIL("decode_attention_static: device %d (at most %d devices)", dev, MAX_DEVICES);
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_of_device[dev]) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      MIE_FAIL("decode_attention_static: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_of_device[dev] = p;
  }
  *ptr = g_scratch_of_device[dev];
  return 0;
}

MIE_EXPORT int mie_decode_attention_static_setup(void) {
  float* p;
  return scratch_for_current_device(&p);
}

MIE_EXPORT long mie_decode_attention_static_capacity(void) { return (long)MIE_DECODE_STATIC_SCRATCH_BYTES; }

MIE_EXPORT int mie_decode_attention_static(const void* q, long q_stride, const void* k_cache, const void* v_cache,
                                           void* out, const int* block_tables, int max_blocks, const int* positions,
                                           int rows, int Hq, int Hkv, int head_dim, int page, float scale, int window,
                                           int partition, int num_splits, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (num_splits <= 1)      // no partial results: the plain entry point allocates nothing either
    return mie_decode_attention(q, q_stride, k_cache, v_cache, out, nullptr, nullptr, block_tables, max_blocks,
                                positions, rows, Hq, Hkv, head_dim, page, scale, window, partition, num_splits, stream);
  if (Hq <= 0 || head_dim != D) MIE_FAIL("decode_attention_static: built for head_dim %d, called with %d (%d heads)", D, head_dim, Hq);
  const size_t entries = (size_t)rows * (size_t)Hq * (size_t)num_splits;
  const size_t need = entries * (D + 1) * sizeof(float);
  if (need > MIE_DECODE_STATIC_SCRATCH_BYTES)
    MIE_FAIL("decode_attention_static: %d rows x %d heads x %d splits x head_dim %d need %zu bytes for partial results; "
             "the library holds %u (fewer splits, or the entry point that takes buffers)",
             rows, Hq, num_splits, D, need, (unsigned)MIE_DECODE_STATIC_SCRATCH_BYTES);
  float* base = nullptr;
  if (scratch_for_current_device(&base)) return -1;
  float* o_part = base;                       // [rows, Hq, splits, D]
  float* lse_part = base + entries * D;       // [rows, Hq, splits]
  return mie_decode_attention(q, q_stride, k_cache, v_cache, out, o_part, lse_part, block_tables, max_blocks, positions,
                              rows, Hq, Hkv, head_dim, page, scale, window, partition, num_splits, stream);
}
