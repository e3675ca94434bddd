// bfloat16 attention over the paged cache for rows of several tokens (prompt portions), on the matrix
// cores of gfx950, for one head size per build (-DHEAD_DIM=N, a multiple of 16 up to 256).
// Caches: keys [pages, Hkv, page, D], values [pages, Hkv, D, page].
//
#include "attention_bf16_common.hpp"

// prefill_attention: rows of several tokens, starting anywhere in their request.  The same two
// products as above with "head" replaced by "query": S^T[key, query] = K . Q^T and
// O^T[d, query] += V^T . P^T, so softmax state is again one value per lane (its query).
//
// A workgroup of PF_WAVES waves serves one kv head and one stretch of 16 QT queries of a row; its waves
// own PF_NT tiles each (16 queries x 1 head; hpw heads by qpw query tiles), waves_h of them side by side
// over the heads of the group and PF_WAVES / waves_h over the queries.  Eight waves of one tile keep two
// waves on every SIMD: the kernel is bound by the number of vector instructions it issues (the softmax;
// head size 64 gives the matrix unit little to do per score), and one wave's waits are the other's turn.
// All waves need the same keys: a block of 32 keys and values is brought into the LDS once by the first
// four waves (two LDS buffers and two sets of registers: block i + 1 waits in registers while block i is
// computed, block i + 2 is on its way, the pages of block i + 3 are looked up), in rows padded so that
// the fragment reads of the matrix instructions meet no bank conflict, values already in the key order
// the second product wants.  Work per stretch grows with its place in the row (causal), so a workgroup
// takes stretch NS - 1 - i and then stretch i: every workgroup of a row has the same number of blocks.
// A block every query of a wave sees whole takes a path without masks; the running maximum m is kept
// in units of scale * log2(e); l is a per-lane partial sum, joined over a query's four lanes at the end.
// Timed alone (one row of 2,048 tokens, 32/4 heads of 64): 61 us, of which about 16 the softmax's vector
// instructions, 14 the fragment reads from the LDS, 10 the matrix instructions, the rest bringing blocks in.
constexpr int PF_WAVES = 8;                         // waves a workgroup
constexpr int PF_NT = 1;                            // tiles a wave owns
constexpr int PF_THREADS = PF_WAVES * 64;
constexpr int PF_KROW = 2 * D + 16;                 // bytes of a key row in the LDS
constexpr int PF_VROW = 2 * BLOCK_KEYS + 16;        // bytes of a value row (one dim, 32 keys) in the LDS
constexpr int PF_KBYTES = BLOCK_KEYS * PF_KROW;
constexpr int PF_BUF = PF_KBYTES + D * PF_VROW;     // one buffer: keys, then values
constexpr int PF_PIECES = 4 * D;                    // 32-byte pieces of a block: 2 D of its keys, then 2 D of its values
constexpr int PF_COPIERS = 256;                     // threads that bring a block in (the first four waves)
constexpr int PF_PPT = (PF_PIECES + PF_COPIERS - 1) / PF_COPIERS;       // pieces such a thread carries

__global__ void __launch_bounds__(PF_THREADS)
prefill_attention_kernel(const bf16* __restrict__ q, long q_stride, const bf16* __restrict__ k_cache,
                         const bf16* __restrict__ v_cache, bf16* __restrict__ out,
                         const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ row_start,
                         const int* __restrict__ row_position, int first_row, int Hq, int Hkv, int hpw,
                         int waves_h, int page, float scale_log2, int window) {
  extern __shared__ __align__(16) unsigned char pf_lds[];
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
  const int qpw = PF_NT / hpw, waves_q = PF_WAVES / waves_h, QT = waves_q * qpw;
  const int head_chunks = (G + hpw * waves_h - 1) / (hpw * waves_h);
  const int kvh = bz / head_chunks, hc = bz - kvh * head_chunks;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, kb = lane >> 4;
  const int t0 = row_start[row], q_len = row_start[row + 1] - t0, p0 = row_position[row];
  const int NS = (q_len + 16 * QT - 1) / (16 * QT);          // stretches of this row
  if (bx >= (NS + 1) / 2) return;               // the whole workgroup, before any barrier
  const int wh = wave % waves_h, wq = wave / waves_h;
  const int* bt = block_tables + (size_t)row * max_blocks;

  for (int pass = 0; pass < 2; ++pass) {
    const int s = pass == 0 ? NS - 1 - bx : bx;
    if (pass == 1 && s >= NS - 1 - bx) break;   // the middle stretch of an odd number has no partner

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

    // ---- bringing a block into the LDS, by the first PF_COPIERS threads (a SIMD then carries one wave that
    // copies and one that does not): a piece is 32 bytes, 16 dims of one key or 16 keys of one dim, so one
    // page look-up and one address serve two loads.  Where a piece lies (page and place in it) is found by
    // walking the block table: [walk_start, walk_start + page) is the page of the block looked up last, and
    // a key at most 31 past a block's start lies at most two pages on.  Addresses are clamped to the row's
    // own keys.
    struct Where {
      int pg[PF_PPT], off[PF_PPT];
    };
    struct Pieces {
      uint4 lo[PF_PPT], hi[PF_PPT];
    };
    const bool copier = tid < PF_COPIERS;
    int walk_idx = blk0 / page, walk_start = walk_idx * page;
    auto lookup = [&](Where& Wh, int blk) {
      if (!copier) return;
      blk = blk < last_blk ? blk : last_blk;           // beyond the last block: the last one again
      while (blk >= walk_start + page) {
        walk_start += page;
        ++walk_idx;
      }
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + PF_COPIERS * i;
        int key;
        if (c < PF_PIECES / 2) {                       // keys: dims 16 j .. 16 j + 15 of key c / (D / 16)
          key = blk + c / (D / 16);
          key = key < kmax ? key : kmax;
        } else {                                       // values: keys 16 g .. 16 g + 15 of one dim, g = c % 2
          key = blk + (c & 1) * 16;
          key = key < (kmax & ~15) ? key : (kmax & ~15);
        }
        const int rel = key - walk_start;
        const int w = (rel >= page ? 1 : 0) + (rel >= 2 * page ? 1 : 0);
        Wh.pg[i] = bt[walk_idx + w];
        Wh.off[i] = rel - w * page;
      }
    };
    auto fetch = [&](Pieces& P, const Where& Wh) {
      if (!copier) return;
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + PF_COPIERS * i;
        const bf16* src = nullptr;
        if (c < PF_PIECES / 2)
          src = k_cache + (((size_t)Wh.pg[i] * Hkv + kvh) * page + Wh.off[i]) * D + (c % (D / 16)) * 16;
        else if (c < PF_PIECES)
          src = v_cache + (((size_t)Wh.pg[i] * Hkv + kvh) * D + ((c - PF_PIECES / 2) >> 1)) * page + Wh.off[i];
        if (src) {
          P.lo[i] = *reinterpret_cast<const uint4*>(src);
          P.hi[i] = *reinterpret_cast<const uint4*>(src + 8);
        }
      }
    };
    auto stash = [&](Pieces& P, int buf, int blk) {
      if (!copier) return;
      unsigned char* base = pf_lds + buf * PF_BUF;
#pragma unroll
      for (int i = 0; i < PF_PPT; ++i) {
        const int c = tid + PF_COPIERS * i;
        if (c < PF_PIECES / 2) {
          unsigned char* at = base + (c / (D / 16)) * PF_KROW + (c % (D / 16)) * 32;
          *reinterpret_cast<uint4*>(at) = P.lo[i];
          *reinterpret_cast<uint4*>(at + 16) = P.hi[i];
        } else if (c < PF_PIECES) {
          const int cv = c - PF_PIECES / 2;
          uint32_t w[8] = {P.lo[i].x, P.lo[i].y, P.lo[i].z, P.lo[i].w, P.hi[i].x, P.hi[i].y, P.hi[i].z, P.hi[i].w};
          const int key0 = blk + (cv & 1) * 16;
          if (key0 + 15 > kmax) {
            // slots after the row's last key may be stale: zero them (0 * NaN must not reach the sum)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              if (key0 + 2 * e > kmax) w[e] &= 0xFFFF0000u;
              if (key0 + 2 * e + 1 > kmax) w[e] &= 0x0000FFFFu;
            }
          }
          // within a row the keys stand in the order the second product wants them: keys 4 g .. 4 g + 3 and
          // 16 + 4 g .. 16 + 4 g + 3 side by side, so that a lane's eight values are one 16-byte read
          unsigned char* at = base + PF_KBYTES + (cv >> 1) * PF_VROW + (cv & 1) * 8;
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) *reinterpret_cast<uint2*>(at + 16 * g4) = make_uint2(w[2 * g4], w[2 * g4 + 1]);
        }
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
        const unsigned char* vr = Vb + (dt * 16 + col) * PF_VROW + 16 * kb;
        va[dt].q = *reinterpret_cast<const uint4*>(vr);
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

    // ---- the blocks, two LDS buffers and two sets of registers: while block i is computed, block i + 1
    // sits in registers (asked for an iteration ago, stored to the LDS after the computing), block i + 2 is
    // on its way from memory and the pages of block i + 3 are looked up.  One barrier a block.
    Where wh;
    Pieces pa, pb;
    lookup(wh, blk0);
    fetch(pa, wh);                                     // block 0
    lookup(wh, blk0 + BLOCK_KEYS);
    fetch(pb, wh);                                     // block 1 (clamped into the row if there is none)
    lookup(wh, blk0 + 2 * BLOCK_KEYS);
    __syncthreads();                                   // the previous stretch is done with the buffers
    stash(pa, 0, blk0);
    __syncthreads();
    auto mine = [&](int blk) { return blk <= wave_kmax && blk + BLOCK_KEYS > wave_kmin; };
    for (int blk = blk0; blk <= kmax; blk += 2 * BLOCK_KEYS) {      // every condition is uniform over the workgroup
      // block blk from buffer 0; pb holds block blk + 32; pa is free for block blk + 64
      if (blk + 2 * BLOCK_KEYS <= kmax) {
        fetch(pa, wh);
        lookup(wh, blk + 3 * BLOCK_KEYS);
      }
      if (mine(blk)) compute(0, blk);
      if (blk + BLOCK_KEYS > kmax) break;              // (no barrier needed: nothing reads the LDS after this)
      stash(pb, 1, blk + BLOCK_KEYS);
      __syncthreads();
      // block blk + 32 from buffer 1; pa holds block blk + 64; pb is free for block blk + 96
      if (blk + 3 * BLOCK_KEYS <= kmax) {
        fetch(pb, wh);
        lookup(wh, blk + 4 * BLOCK_KEYS);
      }
      if (mine(blk + BLOCK_KEYS)) compute(1, blk + BLOCK_KEYS);
      if (blk + 2 * BLOCK_KEYS <= kmax) stash(pa, 0, blk + 2 * BLOCK_KEYS);
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
  int hpw = PF_NT;                       // heads of a kv group per wave: the largest power of two <= min(G, PF_NT)
  while (hpw > G) hpw >>= 1;
  const int head_waves = (G + hpw - 1) / hpw;
  int waves_h = 1;                       // waves side by side over the heads: a power of two up to PF_WAVES
  while (waves_h < head_waves && waves_h < PF_WAVES) waves_h <<= 1;
  const int head_chunks = (G + hpw * waves_h - 1) / (hpw * waves_h);
  const int stretch = (PF_WAVES / waves_h) * (PF_NT / hpw) * 16;      // queries a workgroup serves at a time
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
  dim3 grid((unsigned)gx, rows, Hkv * head_chunks), block(PF_THREADS);
  hipLaunchKernelGGL(prefill_attention_kernel, grid, block, lds_bytes, stream, (const bf16*)q, q_stride,
                     (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, block_tables, max_blocks, row_start,
                     row_position, first_row, Hq, Hkv, hpw, waves_h, page, scale * 1.4426950408889634f, window);
  MIE_CHECK_LAUNCH("prefill_attention");
  return 0;
}
