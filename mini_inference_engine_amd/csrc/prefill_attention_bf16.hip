// bfloat16 attention over the paged cache for rows of several tokens (prompt portions), on the matrix
// cores of gfx950, for one head size per build (-DHEAD_DIM=N, a multiple of 16 up to 256).
// Caches: keys [pages, Hkv, page, D], values [pages, Hkv, D, page].
//
#include "attention_bf16_common.hpp"

// prefill_attention: rows of several tokens, starting anywhere in their request.  With
// v_mfma_f32_32x32x16_bf16 (A: 32 rows x 16 k, B: 16 k x 32 columns, C: 32 x 32, lane l holds column l % 32
// and rows 8 (i / 4) + 4 (l / 32) + i % 4 for i = 0 .. 15)
//   S^T[key, query]  = K[key, d]   . Q^T[d, query]       A = 32 keys x 16 dims from the LDS, B = a query's dims
//   O^T[d, query]   += V^T[d, key] . P^T[key, query]     A = 32 dims x 16 keys from the LDS, B = probabilities
// so a lane owns one query (with one other lane, l ^ 32) and softmax state is one value per lane.  A wave
// owns 32 queries of one head and takes 64 keys a step (two score tiles): per step one maximum, one
// rescaling and one visit of the block's keys and values in the LDS for 2,048 scores.  The scores of a
// lane, taken eight at a time, are already the B operand of the second product if the values' keys stand in
// the matching order in the LDS (16 t + 4 g + {0..3}, 16 t + 8 + 4 g + {0..3} for lane half g), so the
// probabilities never leave registers.
//
// A workgroup of PF_WAVES waves serves one kv head and one stretch of queries of a row: its waves lie side by
// side over the heads of the group and then over 32-query tiles.  All waves need the same keys: a block
// of 64 keys and values is brought into the LDS once by all of them (two LDS buffers and two sets of
// registers: block i + 1 waits in registers while block i is computed, block i + 2 is on its way, the pages
// of block i + 3 are looked up), in rows padded so that the fragment reads meet no bank conflict.  The more
// queries share a block the better: what bounds the kernel at long contexts is the traffic from the L2 into
// the workgroups.  Work per stretch grows with its place in the row (causal), so a workgroup takes stretch
// NS - 1 - i and then stretch i: every workgroup of a row has the same number of blocks.  A block every
// query of a wave sees whole takes a path without masks; the running maximum m is kept in units of
// scale * log2(e); l is a per-lane partial sum, joined over a query's two lanes at the end.
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Waves a workgroup, at head sizes up to 128 (above, eight waves do not fit the registers: always 4):
// 8 over twice the queries (twice the queries share each block that is brought in: at head size 128 and 8,192
// tokens 0.82 against 0.40 PFLOP/s); for rows so short that the grid of 4 waves gives no more workgroups than
// there are compute units, 8 in two halves over the keys on that grid: a wave's chain of blocks is half as
// long and every SIMD has two waves (2,048 tokens at head size 64: 47 against 56 us).  Both kinds of eight
// waves are built and used at every head size up to 128.
constexpr int PF_MAX_WAVES = D > 128 ? 4 : 8;
constexpr int PF_QW = 32;                           // queries a wave owns
constexpr int PF_BK = 64;                           // keys a step
constexpr int KS16 = D / 16;                        // 16-dim steps of q . k
constexpr int DT32 = (D + 31) / 32;                 // 32-dim tiles of the output (the last may be half empty)
constexpr int PF_KROW = 2 * D + 16;                 // bytes of a key row in the LDS
constexpr int PF_VROW = 2 * PF_BK + 16;             // bytes of a value row (one dim, 64 keys) in the LDS
constexpr int PF_KBYTES = PF_BK * PF_KROW;
constexpr int PF_VBYTES = DT32 * 32 * PF_VROW;      // rows of dims beyond D stay zero
constexpr int PF_BUF = PF_KBYTES + PF_VBYTES;       // one buffer: keys, then values
constexpr int PF_KPIECES = PF_BK * (D / 16);        // 32-byte pieces: 16 dims of one key
constexpr int PF_VPIECES = D * (PF_BK / 16);        //                 16 keys of one dim
constexpr int PF_PIECES = PF_KPIECES + PF_VPIECES;

// max of three numbers none of which is a NaN, as one instruction
__device__ __forceinline__ float max3_nn(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// max / sum over the two lanes l, l ^ 32 (one query's lanes)
__device__ __forceinline__ float pair_max(float x) {      // no NaN among the values
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return max_nn(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// KS = 2: the waves form two halves that take the even and the odd 64-key blocks of the same queries (a step
// brings 128 keys in, each half computes its 64) and join their results at the end: half the blocks a wave
// for rows too short to give every SIMD two waves otherwise.
template <int PF_WAVES, int KS>
__global__ void __launch_bounds__(PF_WAVES * 64)
prefill_attention_kernel(const bf16* __restrict__ q, long q_stride, const bf16* __restrict__ k_cache,
                         const bf16* __restrict__ v_cache, bf16* __restrict__ out,
                         const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ row_start,
                         const int* __restrict__ row_position, int first_row, int Hq, int Hkv, int waves_h,
                         int page, float scale_log2, int window) {
  extern __shared__ __align__(16) unsigned char pf_lds[];
  constexpr int PF_THREADS = PF_WAVES * 64;
  constexpr int SUB_WAVES = PF_WAVES / KS;                   // waves of one half
  constexpr int FK = PF_BK * KS;                             // keys a step brings in
  constexpr int T16 = FK / 16;                               // 16-key pieces of a value row a step
  constexpr int KPIECES = KS * PF_KPIECES, PIECES = KS * PF_PIECES;
  constexpr int PF_PPT = (PIECES + PF_THREADS - 1) / PF_THREADS;          // pieces a thread carries
  // Which (stretch pair, row, kv head) this workgroup takes.  Workgroups go to the eight XCDs in turn, in
  // launch order with x fastest, and every XCD has an L2 of its own: all workgroups of one kv head read
  // the same keys and values, so they are placed on one XCD (or on 8 / Z of them when there are fewer
  // than eight z indices), and a block of keys is fetched into one L2 instead of all eight.
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  {
    const unsigned X = gridDim.x, Y = gridDim.y, Z = gridDim.z;
    const unsigned w = blockIdx.x + X * (blockIdx.y + Y * blockIdx.z), total = X * Y * Z;
    if (total % 8 == 0 && (Z % 8 == 0 || 8 % Z == 0)) {       // uniform over the grid
      unsigned r;
      if (Z % 8 == 0) {
        bz = (int)(w % 8 + 8 * ((w / 8) % (Z / 8)));
        r = w / Z;
      } else {
        const unsigned c = w % 8;
        bz = (int)(c % Z);
        r = (w / 8) * (8 / Z) + c / Z;
      }
      bx = (int)(r % X);
      by = (int)(r / X);
    }
  }
  const int row = first_row + by;
  const int G = Hq / Hkv;
  const int waves_q = SUB_WAVES / waves_h;                    // query tiles a workgroup serves at a time
  const int head_chunks = (G + waves_h - 1) / waves_h;
  const int kvh = bz / head_chunks, hc = bz - kvh * head_chunks;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // the same in all lanes: kept in a scalar register
  const int col = lane & 31, g = lane >> 5;
  const int t0 = row_start[row], q_len = row_start[row + 1] - t0, p0 = row_position[row];
  const int STRETCH = PF_QW * waves_q;
  const int NS = (q_len + STRETCH - 1) / STRETCH;              // stretches of this row
  if (bx >= (NS + 1) / 2) return;               // the whole workgroup, before any barrier
  const int wk = wave / SUB_WAVES, wsub = wave - wk * SUB_WAVES;  // which half, and the wave's place in it
  const int wh = wsub % waves_h, wq = wsub / waves_h;
  const int* bt = block_tables + (size_t)row * max_blocks;

  // rows of dims beyond D in the value buffers are never written: zero them once
  if (D % 32 != 0) {
    for (int i = tid; i < 2 * KS * 16 * (PF_VROW / 16); i += PF_THREADS) {
      const int buf = i / (16 * (PF_VROW / 16)), rest = i % (16 * (PF_VROW / 16));
      *reinterpret_cast<uint4*>(pf_lds + buf * PF_BUF + PF_KBYTES + (D + rest / (PF_VROW / 16)) * PF_VROW +
                                (rest % (PF_VROW / 16)) * 16) = make_uint4(0, 0, 0, 0);
    }
  }

  for (int pass = 0; pass < 2; ++pass) {
    const int s = pass == 0 ? NS - 1 - bx : bx;
    if (pass == 1 && s >= NS - 1 - bx) break;   // the middle stretch of an odd number has no partner

    // ---- this wave's tile: 32 queries of one head
    const int gq = hc * waves_h + wh;                          // head within the group
    const int wave_q0 = s * STRETCH + wq * PF_QW;              // first query of the wave
    const bool tile_ok = gq < G && wave_q0 < q_len;
    const int head = kvh * G + (gq < G ? gq : 0);
    int qi = wave_q0 + col;
    const bool q_ok = tile_ok && qi < q_len;
    qi = qi < q_len ? qi : q_len - 1;
    const int qtok = t0 + qi, qpos = p0 + qi;
    const int last_q = wave_q0 + PF_QW - 1 < q_len ? wave_q0 + PF_QW - 1 : q_len - 1;
    const int tile_first = p0 + wave_q0, tile_last = p0 + last_q;
    Frag qf[KS16];
#pragma unroll
    for (int ks = 0; ks < KS16; ++ks) {
      qf[ks].q = make_uint4(0, 0, 0, 0);
      if (tile_ok)
        qf[ks].q = *reinterpret_cast<const uint4*>(q + (size_t)qtok * q_stride + (size_t)head * D + ks * 16 + g * 8);
    }
    // keys the wave's queries can see, and the workgroup's (the union over its waves)
    const int wave_kmax = tile_ok ? tile_last : -1;            // -1: the wave has no query
    const int wave_kmin = window > 0 ? tile_first - window + 1 : 0;
    const int end_q = (s + 1) * STRETCH < q_len ? (s + 1) * STRETCH : q_len;
    const int kmax = p0 + end_q - 1;
    int kmin = window > 0 ? p0 + s * STRETCH - window + 1 : 0;
    kmin = kmin > 0 ? kmin : 0;
    const int blk0 = kmin & ~(PF_BK - 1);
    const int last_blk = kmax & ~(PF_BK - 1);

    float m = -INFINITY, l = 0.f;
    f32x16 O[DT32];
#pragma unroll
    for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) O[dt][i] = 0.f;

    // ---- bringing a block into the LDS, by all threads: a piece is 32 bytes, 16 dims of one key or 16 keys
    // of one dim, so one page look-up and one address serve two loads.  Where a piece lies (page and place
    // in it) is found by walking the block table: [walk_start, walk_start + page) is the page the block looked
    // up last starts in, and a key at most 63 past a block's start lies at most four pages on (pages hold 16
    // keys or more).  Addresses are clamped to the row's own keys.
    struct Where {
      int pg[PF_PPT], off[PF_PPT];
    };
    struct Pieces {
      uint4 lo[PF_PPT], hi[PF_PPT];
    };
    int walk_idx = blk0 / page, walk_start = walk_idx * page;
    // pages of a power of two (the usual 16): a key's page by a shift (the same for every lane)
    const int page_shift = (page & (page - 1)) == 0 ? __builtin_ctz(page) : -1;
    auto lookup = [&](Where& Wh, int blk) {            // blocks are looked up in order, 64 keys apart
      blk = blk < last_blk ? blk : last_blk;           // beyond the last block: the last one again
      {
        const int d = blk - walk_start;
        int adv = 0;
        if (page_shift >= 0) {
          adv = d >> page_shift;
        } else {
#pragma unroll
          for (int k = 1; k <= T16; ++k) adv += d >= k * page ? 1 : 0;
        }
        walk_start += adv * page;
        walk_idx += adv;
      }
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + PF_THREADS * i;
        int key;
        if (c < KPIECES) {                             // keys: dims 16 j .. 16 j + 15 of key c / (D / 16)
          key = blk + c / (D / 16);
          key = key < kmax ? key : kmax;
        } else {                                       // values: keys 16 t .. 16 t + 15 of one dim, t = c % T16
          key = blk + ((c - KPIECES) % T16) * 16;
          key = key < (kmax & ~15) ? key : (kmax & ~15);
        }
        const int rel = key - walk_start;
        int w = 0;
        if (page_shift >= 0) {
          w = rel >> page_shift;
        } else {
#pragma unroll
          for (int k = 1; k <= T16; ++k) w += rel >= k * page ? 1 : 0;
        }
        Wh.pg[i] = bt[walk_idx + w];
        Wh.off[i] = rel - w * page;
      }
    };
    auto fetch = [&](Pieces& P, const Where& Wh) {
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + PF_THREADS * i;
        const bf16* src = nullptr;
        if (c < KPIECES)
          src = k_cache + (((size_t)Wh.pg[i] * Hkv + kvh) * page + Wh.off[i]) * D + (c % (D / 16)) * 16;
        else if (c < PIECES)
          src = v_cache + (((size_t)Wh.pg[i] * Hkv + kvh) * D + (c - KPIECES) / T16) * page + Wh.off[i];
        if (src) {
          P.lo[i] = *reinterpret_cast<const uint4*>(src);
          P.hi[i] = *reinterpret_cast<const uint4*>(src + 8);
        }
      }
    };
    // a set of buffers holds one step: KS blocks of 64 keys, one buffer each
    auto stash = [&](Pieces& P, int set, int blk) {
      unsigned char* base = pf_lds + set * KS * PF_BUF;
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + PF_THREADS * i;
        if (c < KPIECES) {
          const int key = c / (D / 16);
          unsigned char* at = base + (key / PF_BK) * PF_BUF + (key % PF_BK) * PF_KROW + (c % (D / 16)) * 32;
          *reinterpret_cast<uint4*>(at) = P.lo[i];
          *reinterpret_cast<uint4*>(at + 16) = P.hi[i];
        } else if (c < PIECES) {
          const int cv = c - KPIECES, t = cv % T16, dim = cv / T16;
          uint32_t w[8] = {P.lo[i].x, P.lo[i].y, P.lo[i].z, P.lo[i].w, P.hi[i].x, P.hi[i].y, P.hi[i].z, P.hi[i].w};
          const int key0 = blk + t * 16;
          if (key0 + 15 > kmax) {
            // slots after the row's last key may be stale: zero them (0 * NaN must not reach the sum)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              if (key0 + 2 * e > kmax) w[e] &= 0xFFFF0000u;
              if (key0 + 2 * e + 1 > kmax) w[e] &= 0x0000FFFFu;
            }
          }
          // within a row the keys stand in the order the second product wants them: for lane half 0 keys
          // 16 t + {0..3, 8..11}, for lane half 1 keys 16 t + {4..7, 12..15}, each one 16-byte read
          unsigned char* at = base + (t / 4) * PF_BUF + PF_KBYTES + dim * PF_VROW + (t % 4) * 32;
          *reinterpret_cast<uint4*>(at) = make_uint4(w[0], w[1], w[4], w[5]);
          *reinterpret_cast<uint4*>(at + 16) = make_uint4(w[2], w[3], w[6], w[7]);
        }
      }
    };

    // ---- one block of 64 keys for the wave's tile: the wave's half of the step in set `set`
    auto compute = [&](int set, int blk) {
      const unsigned char* Kb = pf_lds + (set * KS + wk) * PF_BUF + col * PF_KROW + g * 16;
      const unsigned char* Vb = pf_lds + (set * KS + wk) * PF_BUF + PF_KBYTES + col * PF_VROW + g * 16;
      f32x16 S[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int i = 0; i < 16; ++i) S[u][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS16; ++ks) {
          Frag a;
          a.q = *reinterpret_cast<const uint4*>(Kb + 32 * u * PF_KROW + ks * 32);
          S[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[ks].v, S[u], 0, 0, 0);
        }
      }
      // every query of the tile sees every key of the block (uniform over the wave)
      const bool whole = blk + PF_BK - 1 <= tile_first && (window <= 0 || blk >= tile_last - window + 1);
      float alpha;
      if (whole) {
        float mx[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          mx[e] = max3_nn(max3_nn(S[0][4 * e], S[0][4 * e + 1], S[0][4 * e + 2]),
                          max3_nn(S[0][4 * e + 3], S[1][4 * e], S[1][4 * e + 1]), max_nn(S[1][4 * e + 2], S[1][4 * e + 3]));
        const float mxx = pair_max(max_nn(max_nn(mx[0], mx[1]), max_nn(mx[2], mx[3])));
        const float m_new = max_nn(m, mxx * scale_log2);
        alpha = fast_exp2(m - m_new);
        m = m_new;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 16; ++i) S[u][i] = fast_exp2(fmaf(S[u][i], scale_log2, -m_new));
      } else {
        const int hi = tile_ok ? qpos : -1;                    // a tile that does not exist sees nothing
        const int lo = window > 0 ? hi - window + 1 : 0;
        float mx = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = blk + 32 * u + 8 * (i >> 2) + 4 * g + (i & 3);
            const bool ok = key >= lo && key <= hi;
            S[u][i] = ok ? S[u][i] : -INFINITY;
            mx = max_nn(mx, S[u][i]);
          }
        mx = pair_max(mx);
        const float m_new = max_nn(m, mx * scale_log2);
        // a query may see none of this block's keys (it lies before the block, or the block before its window)
        alpha = m_new == -INFINITY ? 1.f : fast_exp2(m - m_new);
        m = m_new;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            S[u][i] = S[u][i] == -INFINITY ? 0.f : fast_exp2(fmaf(S[u][i], scale_log2, -m_new));
      }
      float rs = 0.f;
      Frag pb[4];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        float r4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) r4[e] = (S[u][4 * e] + S[u][4 * e + 1]) + (S[u][4 * e + 2] + S[u][4 * e + 3]);
        rs += (r4[0] + r4[1]) + (r4[2] + r4[3]);
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[2 * u + (e >> 2)].w[e & 3] = pack_bf16(S[u][2 * e], S[u][2 * e + 1]);
      }
      l = l * alpha + rs;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {    // the maxima rarely move after the first blocks
#pragma unroll
        for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) O[dt][i] *= alpha;
      }
#pragma unroll
      for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          Frag va;
          va.q = *reinterpret_cast<const uint4*>(Vb + dt * 32 * PF_VROW + t * 32);
          O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va.v, pb[t].v, O[dt], 0, 0, 0);
        }
    };

    // ---- the steps, two sets of LDS buffers and two sets of registers: while step i is computed, step i + 1
    // sits in registers (asked for an iteration ago, stored to the LDS after the computing), step i + 2 is
    // on its way from memory and the pages of step i + 3 are looked up.  One barrier a step.
    Where wh_;
    Pieces pa, pb_;
    lookup(wh_, blk0);
    fetch(pa, wh_);                                    // step 0
    lookup(wh_, blk0 + FK);
    fetch(pb_, wh_);                                   // step 1 (clamped into the row if there is none)
    lookup(wh_, blk0 + 2 * FK);
    __syncthreads();                                   // the previous stretch is done with the buffers
    stash(pa, 0, blk0);
    __syncthreads();
    const int mine_off = wk * PF_BK;                   // this wave's block within a step
    auto mine = [&](int blk) { return blk <= wave_kmax && blk + PF_BK > wave_kmin; };
    for (int blk = blk0; blk <= kmax; blk += 2 * FK) {         // every condition is uniform over the workgroup
      // step blk from set 0; pb_ holds step blk + FK; pa is free for step blk + 2 FK
      if (blk + 2 * FK <= kmax) {
        fetch(pa, wh_);
        lookup(wh_, blk + 3 * FK);
      }
      if (mine(blk + mine_off)) compute(0, blk + mine_off);
      if (blk + FK > kmax) break;
      stash(pb_, 1, blk + FK);
      __syncthreads();
      // step blk + FK from set 1; pa holds step blk + 2 FK; pb_ is free for step blk + 3 FK
      if (blk + 3 * FK <= kmax) {
        fetch(pb_, wh_);
        lookup(wh_, blk + 4 * FK);
      }
      if (mine(blk + FK + mine_off)) compute(1, blk + FK + mine_off);
      if (blk + 2 * FK <= kmax) stash(pa, 0, blk + 2 * FK);
      __syncthreads();
    }

    if (KS == 2) {
      // The halves join: the second half's state goes through the LDS (item i of lane l at 4 (64 i + l), a
      // region a wave), the first half rescales both to the common maximum.  l and O are per-lane partial
      // sums, m is the same in a query's two lanes.
      static_assert(KS == 1 || SUB_WAVES * 64 * (2 + 16 * DT32) * 4 <= 2 * KS * PF_BUF, "the halves' exchange must fit the buffers");
      float* xch = reinterpret_cast<float*>(pf_lds) + wsub * (64 * (2 + 16 * DT32)) + lane;
      __syncthreads();                                 // everybody is done with the keys and values
      if (wk == 1) {
        xch[0] = m;
        xch[64] = l;
#pragma unroll
        for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) xch[64 * (2 + dt * 16 + i)] = O[dt][i];
      }
      __syncthreads();
      if (wk == 0) {
        const float m1 = xch[0], l1 = xch[64];
        const float mj = max_nn(m, m1);
        // a half may have seen no key of a query (m = -inf, sums 0): it counts for nothing
        const float a0 = m == -INFINITY ? 0.f : fast_exp2(m - mj);
        const float a1 = m1 == -INFINITY ? 0.f : fast_exp2(m1 - mj);
        l = l * a0 + l1 * a1;
#pragma unroll
        for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) O[dt][i] = O[dt][i] * a0 + xch[64 * (2 + dt * 16 + i)] * a1;
      }
    }

    const float total = pair_sum(l);
    if (q_ok && wk == 0) {
      const float inv = 1.0f / total;
      bf16* op = out + ((size_t)qtok * Hq + head) * D + 4 * g;
#pragma unroll
      for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int d0 = dt * 32 + 8 * e;              // this lane's dims d0 + 4 g .. + 3
          if (d0 < D) {
            uint2 st;
            st.x = pack_bf16(O[dt][4 * e] * inv, O[dt][4 * e + 1] * inv);
            st.y = pack_bf16(O[dt][4 * e + 2] * inv, O[dt][4 * e + 3] * inv);
            *reinterpret_cast<uint2*>(op + d0) = st;
          }
        }
    }
  }
}

MIE_EXPORT const char* prefill_attention_bf16_last_error() { return g_mie_error; }

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
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) MIE_FAIL("prefill_attention: no current device");
  static int compute_units[64] = {};              // of each device, asked for once
  if (compute_units[dev] <= 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      MIE_FAIL("prefill_attention: cannot read the number of compute units of device %d", dev);
    compute_units[dev] = n;
  }
  // the grid for `waves` waves a workgroup: waves side by side over the heads of a group (a power of two), the rest
  // over 32-query tiles; a workgroup takes a late stretch and an early one
  auto plan = [&](int waves, int* waves_h, dim3* grid) {
    int wh = 1;
    while (wh < G && wh < waves) wh <<= 1;
    const int head_chunks = (G + wh - 1) / wh;
    const int stretch = (waves / wh) * PF_QW;
    const long stretches = (max_row_tokens + stretch - 1) / stretch;
    *waves_h = wh;
    *grid = dim3((unsigned)((stretches + 1) / 2), rows, Hkv * head_chunks);
    return (long)grid->x * grid->y * grid->z;
  };
  // Eight waves over twice the queries where that still gives every compute unit a workgroup; else, at head
  // sizes that leave room, eight waves in two halves over the keys (the grid of four waves); else four waves.
  enum { FOUR, EIGHT_QUERIES, EIGHT_KEYS } kind = FOUR;
  int waves_h;
  dim3 grid;
  if (PF_MAX_WAVES == 8) {
    // A compute unit holds one workgroup of eight waves (registers): more of the two-halves kind than compute
    // units would run in two rounds, the second half empty (2,560 tokens: 95 us, against 45 for 2,048).
    const long n4 = plan(4, &waves_h, &grid);
    kind = n4 > compute_units[dev] ? EIGHT_QUERIES : EIGHT_KEYS;
  }
  plan(kind == EIGHT_QUERIES ? 8 : 4, &waves_h, &grid);
  if (grid.y > 65535 || grid.z > 65535) MIE_FAIL("prefill_attention: grid too large (%d rows)", rows);
  const float scale_log2 = scale * 1.4426950408889634f;
  // more LDS than a kernel gets by default is asked for once per kernel and device
  static bool lds_allowed[3][64] = {};
  auto launch = [&](auto kernel, int waves, int lds_bytes) -> int {
    if (lds_bytes > 64 * 1024 && !lds_allowed[kind][dev]) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) MIE_FAIL("prefill_attention: %d bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
      lds_allowed[kind][dev] = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(waves * 64), lds_bytes, stream, (const bf16*)q, q_stride, (const bf16*)k_cache,
                       (const bf16*)v_cache, (bf16*)out, block_tables, max_blocks, row_start, row_position, first_row, Hq, Hkv,
                       waves_h, page, scale_log2, window);
    return 0;
  };
  int rc = 0;
  if constexpr (PF_MAX_WAVES == 8) {
    if (kind == EIGHT_QUERIES) rc = launch(prefill_attention_kernel<8, 1>, 8, 2 * PF_BUF);
    if (kind == EIGHT_KEYS) rc = launch(prefill_attention_kernel<8, 2>, 8, 4 * PF_BUF);
  }
  if (kind == FOUR) rc = launch(prefill_attention_kernel<4, 1>, 4, 2 * PF_BUF);
  if (rc) return rc;
  MIE_CHECK_LAUNCH("prefill_attention");
  return 0;
}
