// Window-bounded single-query attention, split-K, bf16/fp16, matrix-core version.
//
// Why matrix cores here: with a GQA group of 7 every K/V byte feeds 7 query heads, i.e. 7 flop per
// byte; done on the vector ALUs that is ~900 VALU instructions per 16-key tile and the split kernel
// ran VALU-bound (71 % VALU issue utilisation at 50 % of HBM peak on the 7B decode shape). The
// group is therefore padded to the 16-wide N dimension of v_mfma_f32_16x16x32 and both
// contractions run on the matrix cores; what is left on the VALU is the softmax of a
// [32 keys x 16 heads] tile (8 values per lane) and an in-register 8x8 transpose of V.
//
// Work decomposition: grid = (query rows, kv-head groups, splits). A workgroup has one wavefront
// per kv head (up to 8), all walking the same part of the same sequence's window: the heads of a
// cache row are adjacent in memory (a 16-token block of 4 heads is 16 KiB contiguous), so the
// wavefronts of a workgroup together stream whole DRAM pages instead of 256-byte pieces 1 KiB
// apart. Wavefronts are independent (own head group, own online softmax, own partial result):
// no LDS, no barrier. A wavefront walks over "chunks" of 32 keys (two 16-key tiles).
// Lane = (g = lane/16, c = lane%16). K/V are read once, with non-temporal loads.
//
//   S^T = K Q^T   A = K tile  : lane (g,c) holds key c of the tile, dims of 16-byte chunk 4s+g
//                 B = Q^T     : lane (g,c) holds head c (zero for c >= G), same dims
//                 D = S^T     : lane (g,c) holds head c, keys 4g..4g+3 of the tile
//   O^T = V^T P^T A = V^T     : lane (g,c) holds dim 8c+mt, keys kk = 8g..8g+7 of the chunk, where
//                               kk = 8g+j is key 4g+j of tile 0 (j<4) or key 4g+j-4 of tile 1
//                 B = P^T     : lane (g,c) holds head c, the same 8 keys: exactly the S^T results of
//                               that lane, so P never leaves its registers
//                 D = O^T     : lane (g,c) holds head c, dims 32g + 8i + mt (i<4, mt<8)
//   V is loaded as 16-byte row pieces (lane (g,c): its 8 keys, dims 8c..8c+7; one instruction covers
//   4 whole 256-byte rows) and the 8x8 (key x dim) block of a lane is transposed in registers with
//   v_perm_b32 to give the 8 A operands. K loads cover 16 rows x 64 bytes per instruction.
//   Softmax state (running max m, denominator l) is per lane for head c; the max is shared by the
//   four g groups of a head through two cross-lane exchanges per chunk.
// Rows outside [lo, hi) are never read: row indices are clamped into the visible range for the
// address and masked by their true index for the score, so stale or uninitialised cache rows
// cannot leak NaNs through 0 * NaN.
#include <type_traits>

#include <hip/hip_ext.h>

#include "common.h"
#include "mfma_util.h"
#include "swa_decode_params.h"

namespace {

using namespace sb;

constexpr float kNegInf = kNegInfF;

struct Chunk {
  uint4 k0[4], k1[4];  // K operands of tile 0 / tile 1, one per 32-dim step
  uint4 v[8];          // V rows of this lane's 8 keys, dims 8c..8c+7
};

// Visible keys [lo, hi) of query row r and the 32-key chunks they touch: returns their number,
// `first_chunk` = index of the first.
__device__ __forceinline__ int row_chunks(const DecodeParams &p, const int32_t *seq_lens, int64_t r, int &lo, int &hi,
                                          int &first_chunk) {
  hi = seq_lens[r];
  lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
  if (p.key_lo) lo = max(lo, p.key_lo[r]);
  first_chunk = lo >> 5;
  return hi > lo ? ((hi - 1) >> 5) - first_chunk + 1 : 0;
}

// One wavefront's work on chunks [cb, ce) of row r for kv head kvh: attention over those keys
// with an online softmax of its own, result written as the row's output (`direct`) or as the
// fp32 partial number part_base + head * part_hs. kDepth = chunks in flight besides the one being
// computed. `owns_newest`: this range ends the row's window (with a fused append it stores the
// step's K/V row into the cache). Meta tokens: the call also takes chunks meta_first,
// meta_first + meta_step, ... of the p.meta_len shared meta rows into the same softmax (meta_step 0:
// none); the first of them is fetched before the window is walked and computed after it.
template <typename E, int kDepth, int kLookups, bool kMergeHere = false>
__device__ __forceinline__ void split_segment(const DecodeParams &p, const int32_t *block_table, const int G,
                                              const int kvh, const int lane, const int64_t r, const int lo,
                                              const int hi, const int cb, const int ce, const bool owns_newest,
                                              const bool direct, const int64_t part_base, const int part_hs,
                                              const int meta_first, const int meta_step) {
  const int g = lane >> 4;
  const int c = lane & 15;
  const int64_t seq = p.row_seq ? (int64_t)p.row_seq[r] : r;
  const bool any = hi > lo;
  const int first_tile = lo >> 4;
  const int last_tile = any ? (hi - 1) >> 4 : first_tile;

  // Q^T operands: head c of the group, dims of chunk 4s+g; zero rows pad the group to 16 heads
  uint4 qb[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    qb[s] = make_uint4(0u, 0u, 0u, 0u);
    if (c < G)
      qb[s] = *reinterpret_cast<const uint4 *>(
          p.q + (r * p.q_sr + (int64_t)(kvh * G + c) * p.q_sh + (4 * s + g) * 8) * 2);
  }

  const float my_slope = (p.opt.slopes && c < G) ? p.opt.slopes[kvh * G + c] : 0.f;  // ALiBi slope of this lane's head

  f32x4_t acc[8];
#pragma unroll
  for (int mt = 0; mt < 8; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = kNegInf, l = 0.f;

  const bool paged = block_table != nullptr;
  const int64_t dense_row0 = (!paged && p.kv_start) ? p.kv_start[seq] : 0;
  const int64_t head_off = (int64_t)kvh * p.kv_sh;

  // byte offset of row 0 of tile t (t inside [first_tile, last_tile]; uniform over the wavefront)
  auto tile_base = [&](int t) -> int64_t {
    const int i0 = t << 4;
    if (paged) {
      const int bi = i0 / p.block_size;
      const int64_t blk = block_table[seq * p.bt_stride + bi];
      return blk * p.kv_sb + (int64_t)(i0 - bi * p.block_size) * p.kv_sr + head_off;
    }
    return (dense_row0 + i0) * p.kv_sr + head_off;
  };
  // the same for six tiles at once, under ONE paged/dense branch: the six table lookups are then
  // independent loads of one block and cost one round trip (one tile_base call after another, each with
  // its own branch, waits for every lookup before making the next)
  auto tile_bases6 = [&](const int (&t)[6], int64_t (&base)[6]) {
    if (paged) {
      int bi[6];
      int64_t blk[6];
#pragma unroll
      for (int n = 0; n < 6; ++n) bi[n] = (t[n] << 4) / p.block_size;
      // kLookups = 1: written out as one block of scalar loads and one wait; left to itself (kLookups = 0) the
      // compiler, short of scalar registers here, issues each load only after the previous one has
      // returned: six round trips before the first K/V load. Not in the balanced kernel: handing the table
      // pointer to an asm statement counts as letting it escape, the no-alias guarantee against that
      // kernel's partial stores is gone, and the lookups of its streaming loop turn into vector loads
      // (measured 12 % slower). There (kLookups = 2) lanes 0..5 fetch one entry each with ONE vector load
      // (nothing else is in flight at the start of a segment, so it waits for nothing but itself) and
      // the six values are read back across lanes.
      if constexpr (kLookups == 0) {
#pragma unroll
        for (int n = 0; n < 6; ++n) blk[n] = block_table[seq * p.bt_stride + bi[n]];
      } else if constexpr (kLookups == 2) {
        int mine = bi[0];
#pragma unroll
        for (int n = 1; n < 6; ++n) mine = lane == n ? bi[n] : mine;
        const int32_t e = block_table[seq * p.bt_stride + mine];
#pragma unroll
        for (int n = 0; n < 6; ++n) blk[n] = __builtin_amdgcn_readlane(e, n);
      } else {
      const int32_t *row = block_table + seq * p.bt_stride;
      const int32_t *a0 = row + bi[0], *a1 = row + bi[1], *a2 = row + bi[2], *a3 = row + bi[3], *a4 = row + bi[4],
                    *a5 = row + bi[5];
      int32_t e0, e1, e2, e3, e4, e5;
      asm(  // not volatile: a volatile asm counts as a possible store and would do the same
          "s_load_dword %0, %6, 0x0\n\t"
          "s_load_dword %1, %7, 0x0\n\t"
          "s_load_dword %2, %8, 0x0\n\t"
          "s_load_dword %3, %9, 0x0\n\t"
          "s_load_dword %4, %10, 0x0\n\t"
          "s_load_dword %5, %11, 0x0\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&s"(e0), "=&s"(e1), "=&s"(e2), "=&s"(e3), "=&s"(e4), "=&s"(e5)
          : "s"(a0), "s"(a1), "s"(a2), "s"(a3), "s"(a4), "s"(a5));  // (reads only: no memory clobber, which
                                                                      // would turn later lookups into vector loads)
      blk[0] = e0; blk[1] = e1; blk[2] = e2; blk[3] = e3; blk[4] = e4; blk[5] = e5;
      }
#pragma unroll
      for (int n = 0; n < 6; ++n)
        base[n] = blk[n] * p.kv_sb + (int64_t)((t[n] << 4) - bi[n] * p.block_size) * p.kv_sr + head_off;
    } else {
#pragma unroll
      for (int n = 0; n < 6; ++n) base[n] = (dense_row0 + (t[n] << 4)) * p.kv_sr + head_off;
    }
  };
  auto clamp_tile = [&](int t) { return min(max(t, first_tile), last_tile); };
  // row of tile tc whose key index is the visible key nearest to (tc*16 + row)
  auto clamp_row = [&](int tc, int row) { return min(max((tc << 4) + row, lo), hi - 1) - (tc << 4); };

  // Lane offsets inside a tile (bytes, 32-bit): K row c at 16-byte piece g; V rows 4g+j at piece c.
  // Interior chunks use these constants; edge chunks (first/last of the window) clamp their rows.
  const uint32_t kv_sr32 = (uint32_t)p.kv_sr;
  const uint32_t koff = c * kv_sr32 + g * 16;
  uint32_t voff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) voff[j] = (4 * g + j) * kv_sr32 + c * 16;

  // Fused append: the newest key (index hi-1) is not in the cache yet. Its K/V rows are read from
  // the step's key/value tensors wherever a lane's (clamped) row is hi-1, and the wavefront that
  // owns the last chunk of the window stores them into the cache slot at the very end of the
  // kernel. (The store must stay behind every block-table lookup: a global store ahead of them
  // would stop the compiler from proving the table unclobbered, the lookups would turn from
  // scalar loads into vector loads, and each would then wait for all K/V loads in flight.)
  const bool fused = p.new_k != nullptr;
  const char *newk = fused ? p.new_k + r * p.nk_st + (int64_t)kvh * p.nk_sh : nullptr;
  const char *newv = fused ? p.new_v + r * p.nv_st + (int64_t)kvh * p.nv_sh : nullptr;
  // ---- loaders ---------------------------------------------------------------------------
  // Interior chunk (every key visible): wave-uniform bases plus constant 32-bit lane offsets.
  auto load_interior = [&](int64_t b0, int64_t b1, Chunk &ck) {
    const char *k0p = p.k + b0, *k1p = p.k + b1, *v0p = p.v + b0, *v1p = p.v + b1;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      ck.k0[s] = load_stream16(k0p + koff + s * 64);
      ck.k1[s] = load_stream16(k1p + koff + s * 64);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ck.v[j] = load_stream16(v0p + voff[j]);
      ck.v[4 + j] = load_stream16(v1p + voff[j]);
    }
  };
  // Edge chunk (first / last chunk of the window; also correct for any other chunk): per-lane
  // pointers, tiles and rows clamped into the visible range, the newest row taken from the step
  // inputs when the append is fused. base0/base1 = the bases of tiles clamp_tile(2cc), clamp_tile(2cc+1):
  // the block-table lookups are made apart from the loads, all of a segment's in one go (tile_bases6).
  auto load_edge = [&](int cc, int64_t base0, int64_t base1, Chunk &ck) {
    const int t0c = clamp_tile(2 * cc), t1c = clamp_tile(2 * cc + 1);
    const char *k0p = p.k + base0, *k1p = p.k + base1;
    const char *v0p = p.v + (k0p - p.k), *v1p = p.v + (k1p - p.k);
    const int newest = fused ? hi - 1 : -1;
    const int r0 = clamp_row(t0c, c), r1 = clamp_row(t1c, c);
    const char *pk0 = ((t0c << 4) + r0 == newest) ? newk + g * 16 : k0p + r0 * kv_sr32 + g * 16;
    const char *pk1 = ((t1c << 4) + r1 == newest) ? newk + g * 16 : k1p + r1 * kv_sr32 + g * 16;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      ck.k0[s] = load_stream16(pk0 + s * 64);
      ck.k1[s] = load_stream16(pk1 + s * 64);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int q0 = clamp_row(t0c, 4 * g + j), q1 = clamp_row(t1c, 4 * g + j);
      ck.v[j] = load_stream16(((t0c << 4) + q0 == newest) ? newv + c * 16 : v0p + q0 * kv_sr32 + c * 16);
      ck.v[4 + j] = load_stream16(((t1c << 4) + q1 == newest) ? newv + c * 16 : v1p + q1 * kv_sr32 + c * 16);
    }
  };

  // Meta chunk cc: rows 32cc .. 32cc+31 of the dense meta tensors, clamped to the last row (masked by
  // their true index in the scores). Ordinary loads: every workgroup of the launch reads these rows.
  auto load_meta = [&](int cc, Chunk &ck) {
    const char *mk = p.meta_k + (int64_t)kvh * p.meta_sh, *mv = p.meta_v + (int64_t)kvh * p.meta_sh;
    const int last = p.meta_len - 1, i0 = cc << 5;
    const char *pk0 = mk + (int64_t)min(i0 + c, last) * p.meta_sr + g * 16;
    const char *pk1 = mk + (int64_t)min(i0 + 16 + c, last) * p.meta_sr + g * 16;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      ck.k0[s] = *reinterpret_cast<const uint4 *>(pk0 + s * 64);
      ck.k1[s] = *reinterpret_cast<const uint4 *>(pk1 + s * 64);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ck.v[j] = *reinterpret_cast<const uint4 *>(mv + (int64_t)min(i0 + 4 * g + j, last) * p.meta_sr + c * 16);
      ck.v[4 + j] = *reinterpret_cast<const uint4 *>(mv + (int64_t)min(i0 + 16 + 4 * g + j, last) * p.meta_sr + c * 16);
    }
  };

  // One chunk of work: S^T = K Q^T, online softmax, O^T += V^T P^T. kMask = edge chunk (keys outside
  // [mlo, mhi) are masked by their true index).
  auto compute_chunk = [&](int ch, const Chunk &ck, auto mask_tag, const int mlo, const int mhi, auto meta_tag) {
    constexpr bool kMask = decltype(mask_tag)::value;
    constexpr bool kMeta = decltype(meta_tag)::value;  // a chunk of meta rows: their ALiBi term has its own distance
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      s0 = Mma<E>::run(ck.k0[s], qb[s], s0);
      s1 = Mma<E>::run(ck.k1[s], qb[s], s1);
    }
    float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
    if (p.opt.on) {  // soft cap / ALiBi (wave-uniform; the query sits at key index hi - 1)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = (ch << 5) + ((j >> 2) << 4) + 4 * g + (j & 3);
        const float dist = kMeta ? -fabsf((float)(p.meta_bias_off + (int)r - key)) : (float)(key - (hi - 1));
        sc[j] = adjust_score(p.opt, sc[j], my_slope, dist);
      }
    }
    if constexpr (kMask) {
      const int i0 = ch << 5;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int i = i0 + ((j >> 2) << 4) + 4 * g + (j & 3);
        if (i < mlo || i >= mhi) sc[j] = kNegInf;
      }
    }
    float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m, mx * p.scale_log2);
    const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = fast_exp2(m - m_safe);
    const bool grew = m_new > m;
    m = m_new;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      sc[j] = fast_exp2(fmaf(sc[j], p.scale_log2, -m_safe));
      psum += sc[j];
    }
    l = fmaf(l, alpha, psum);
    if (__builtin_amdgcn_ballot_w64(grew) != 0) {
#pragma unroll
      for (int mt = 0; mt < 8; ++mt) acc[mt] *= alpha;
    }
    const uint4 pb = make_uint4(Mma<E>::pack(sc[0], sc[1]), Mma<E>::pack(sc[2], sc[3]),
                                Mma<E>::pack(sc[4], sc[5]), Mma<E>::pack(sc[6], sc[7]));
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
      const int w = mt >> 1;
      uint4 vt;
      if (mt & 1) {
        vt = make_uint4(perm_hi(word(ck.v[1], w), word(ck.v[0], w)), perm_hi(word(ck.v[3], w), word(ck.v[2], w)),
                        perm_hi(word(ck.v[5], w), word(ck.v[4], w)), perm_hi(word(ck.v[7], w), word(ck.v[6], w)));
      } else {
        vt = make_uint4(perm_lo(word(ck.v[1], w), word(ck.v[0], w)), perm_lo(word(ck.v[3], w), word(ck.v[2], w)),
                        perm_lo(word(ck.v[5], w), word(ck.v[4], w)), perm_lo(word(ck.v[7], w), word(ck.v[6], w)));
      }
      acc[mt] = Mma<E>::run(vt, pb, acc[mt]);
    }
  };
  const std::true_type kMasked{};
  const std::false_type kUnmasked{};

  // Only the first and the last chunk of a window can hold keys outside [lo, hi). They are taken
  // out of the streaming loop: their loads go into registers of their own and they are computed
  // before / after the loop, so the loop body has no clamping, no masking and a fixed number of
  // loads in flight. The loop is a software pipeline kDepth chunks deep over a ring of kDepth+1
  // register sets (unrolled over the ring, no register copies); prefetches past the end re-read
  // the last interior chunk; tile bases (block-table lookups) run one chunk ahead of the loads.
  // Interior chunks lie wholly inside [lo, hi), so the unclamped interior loader (and the block
  // table lookups made for it) never leave the sequence; when a split has no interior chunk the
  // loop and its prologue are skipped altogether.
  const int meta_chunks = (p.meta_len + 31) >> 5;
  const bool has_meta = meta_step > 0 && meta_first < meta_chunks;
  Chunk metac;
  if (has_meta) load_meta(meta_first, metac);

  if (cb < ce) {
    // with a fused append the chunk holding the newest key is an edge chunk even when it is full:
    // that row is not in the cache yet and only the edge loader reads it from the step inputs
    auto is_edge = [&](int cc) {
      return (cc << 5) < lo || (cc << 5) + 32 > hi || (fused && cc == ((hi - 1) >> 5));
    };
    const bool e_head = is_edge(cb);
    const bool e_tail = (ce - 1 > cb) && is_edge(ce - 1);
    const int ib = cb + (e_head ? 1 : 0), ie = ce - (e_tail ? 1 : 0);  // interior chunks [ib, ie)
    // An edge chunk is fetched only where the segment has one (a window cut into n parts has two among
    // its 2n ends), the head first because it is computed first, the tail two chunks before the stream
    // ends: fetched up front it only delayed every workgroup's first chunks, all workgroups asking at once.
    // The table lookups of both are made here, together with the first interior one.
    Chunk head, tail;
    const int tiles6[6] = {clamp_tile(2 * cb),       clamp_tile(2 * cb + 1),       // head chunk
                           clamp_tile(2 * (ce - 1)), clamp_tile(2 * (ce - 1) + 1), // tail chunk
                           clamp_tile(2 * ib),       clamp_tile(2 * ib + 1)};      // first interior chunk
    int64_t base6[6];
    tile_bases6(tiles6, base6);
    const int64_t hb0 = base6[0], hb1 = base6[1], tb0 = base6[2], tb1 = base6[3];
    if (ib < ie) {
      const int lastc = ie - 1;
      int64_t b0, b1;
      auto locate = [&](int cc) {
        b0 = tile_base(2 * cc);
        b1 = tile_base(2 * cc + 1);
      };
      // loads chunk min(cc, lastc), whose tiles the previous call located, and locates the next one
      auto issue = [&](int cc, Chunk &dst) {
        const int64_t lb0 = b0, lb1 = b1;
        locate(min(cc + 1, lastc));
        load_interior(lb0, lb1, dst);
      };
      Chunk ring[kDepth + 1];
      int ch = ib;
      b0 = base6[4];
      b1 = base6[5];
      if (e_head) load_edge(cb, hb0, hb1, head);
#pragma unroll
      for (int u = 0; u < kDepth; ++u) issue(ch + u, ring[u]);
      if (e_head) compute_chunk(cb, head, kMasked, lo, hi, kUnmasked);
      const int tail_at = e_tail ? max(ib, ie - 2) : -1;
      bool more = true;
      while (more) {
#pragma unroll
        for (int u = 0; u <= kDepth; ++u) {
          if (more) {
            if (ch == tail_at) load_edge(ce - 1, tb0, tb1, tail);
            issue(ch + kDepth, ring[(u + kDepth) % (kDepth + 1)]);
            compute_chunk(ch, ring[u], kUnmasked, lo, hi, kUnmasked);
            ++ch;
            more = ch < ie;
          }
        }
      }
    } else {
      if (e_head) load_edge(cb, hb0, hb1, head);
      if (e_tail) load_edge(ce - 1, tb0, tb1, tail);
      if (e_head) compute_chunk(cb, head, kMasked, lo, hi, kUnmasked);
    }
    if (e_tail) compute_chunk(ce - 1, tail, kMasked, lo, hi, kUnmasked);
  }

  if (has_meta) {
    compute_chunk(meta_first, metac, kMasked, 0, p.meta_len, kMasked);
    for (int cc = meta_first + meta_step; cc < meta_chunks; cc += meta_step) {
      load_meta(cc, metac);
      compute_chunk(cc, metac, kMasked, 0, p.meta_len, kMasked);
    }
  }

  // ---- fused append: store the newest K/V row at its slot ---------------------------------
  if (fused && any && owns_newest && cb < ce && lane < 32) {
    const int64_t slot = p.slot_mapping[r];
    if (slot >= 0) {
      const int64_t blk = slot / p.block_size;
      const int64_t dst = blk * p.kv_sb + (slot - blk * p.block_size) * p.kv_sr + head_off + (lane & 15) * 16;
      if (lane < 16)
        *reinterpret_cast<uint4 *>(const_cast<char *>(p.k) + dst) = *reinterpret_cast<const uint4 *>(newk + lane * 16);
      else
        *reinterpret_cast<uint4 *>(const_cast<char *>(p.v) + dst) = *reinterpret_cast<const uint4 *>(newv + (lane & 15) * 16);
    }
  }

  // ---- denominators of the four g groups -> one per head ------------------------------
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);

  // ---- this wavefront's result: lane (g, c < G) owns head c, dims 32g + 8i + mt --------------
  if (c < G) {
    const int hq = kvh * G + c;
    if (direct) {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      char *dst = p.out + (r * p.o_sr + (int64_t)hq * p.o_sh + 32 * g) * 2;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint4 o;
        o.x = E::pack(acc[0][i] * inv, acc[1][i] * inv);
        o.y = E::pack(acc[2][i] * inv, acc[3][i] * inv);
        o.z = E::pack(acc[4][i] * inv, acc[5][i] * inv);
        o.w = E::pack(acc[6][i] * inv, acc[7][i] * inv);
        *reinterpret_cast<uint4 *>(dst + 16 * i) = o;
      }
      if (g == 0 && p.lse) p.lse[r * p.Hq + hq] = l > 0.f ? (m + log2f(l)) * kLn2 : kNegInf;
    } else {
      const int64_t part = part_base + (int64_t)hq * part_hs;
      float *dst = p.ws_acc + part * 128 + 32 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        reinterpret_cast<float4 *>(dst + 8 * i)[0] = make_float4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]);
        reinterpret_cast<float4 *>(dst + 8 * i)[1] = make_float4(acc[4][i], acc[5][i], acc[6][i], acc[7][i]);
      }
      if (g == 0) {
        p.ws_ml[part * 2] = m;
        p.ws_ml[part * 2 + 1] = l;
      }
    }
  }

  // ---- merge by the last wavefront of the row to arrive ------------------------------------------------
  // The n_split wavefronts that work on (row r, kv head kvh) run in workgroups whose numbers differ by
  // multiples of 8 (the launch pads the row count to a multiple of 8), and workgroup i of a launch runs on
  // XCD i % 8: they all sit behind ONE L2. Inside an XCD the L2 is the point of coherence, so handing the
  // partials from one wavefront to another takes no cache write-back: a wavefront waits until its own
  // partial stores have been acknowledged by the L2, then bumps the pair's counter (an atomic executed in
  // that L2); whoever sees n_split - 1 knows that every partial of the pair is in the L2, reads them with
  // loads that skip its CU's L1 (sc1), merges exactly as swa_decode_merge_kernel does (same order, same
  // arithmetic: the same bits) and zeroes the counter for the next launch. Nobody waits for anybody.
  // (Across XCDs the same hand-over needs the dirty L2 lines written back to memory and the reader's L2
  // invalidated: with agent-scope fences that made the whole step 1.5x slower.)
  // Measured on the 7B decode shape (64 rows x 4 splits): the chain partial stores acknowledged -> counter ->
  // partial loads -> output stores at the end of the last wavefront costs 5.7 us of kernel time, against
  // 4.8 us for the merge kernel plus its launch gap: no gain (88 -> 94 us per step), and none at 16, 32 or 128
  // rows either. The variant is therefore opt-in (SB_DECODE_MERGE_IN_KERNEL); it is an instantiation of its
  // own so that its 160 extra live registers do not weigh on the default kernel.
  if constexpr (kMergeHere) if (!direct && p.merge_counter != nullptr) {
    // this wavefront's partial stores must have been acknowledged by the L2 before the counter moves: an
    // explicit wait (a workgroup-scope release fence alone need not wait for vector stores), with the fence
    // kept as a barrier for the compiler's own reordering
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), expcnt and lgkmcnt left alone (gfx9 encoding)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    int *counter = p.merge_counter + r * p.Hkv + kvh;
    const int xcc = (int)__builtin_amdgcn_s_getreg(20 | (3 << 11));  // HW_REG_XCC_ID, bits 3:0
    int arrived = 0;
    if (lane == 0) arrived = __hip_atomic_fetch_add(counter, 1 + (xcc << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // (orders the compiler; the loads below skip the L1 themselves)
    if ((arrived & 0xff) != p.n_split - 1) return;
    if (lane == 0) {
      *counter = 0;
      // every contributor must have run on this XCD; if not, the sticky fault word (last counter) says so
      if ((arrived >> 8) + xcc != p.n_split * xcc) p.merge_counter[kMergeFaultWord] = 1;
    }
    if (c >= G) return;
    const int hq = kvh * G + c;
    const int64_t part0 = (r * p.Hq + hq) * (int64_t)p.n_split;
    const __amdgpu_buffer_rsrc_t acc_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.ws_acc, 0, 0x7fffffff, 0x00020000);
    float tot[32];
#pragma unroll
    for (int d = 0; d < 32; ++d) tot[d] = 0.f;
    float L = 0.f, M = kNegInf;
    for (int s0 = 0; s0 < p.n_split; s0 += 4) {
      float ms[4], ls[4];
      u32x4_t av[4][8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t part = part0 + min(s0 + j, p.n_split - 1);
        ms[j] = __hip_atomic_load(p.ws_ml + part * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ls[j] = __hip_atomic_load(p.ws_ml + part * 2 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int q4 = 0; q4 < 8; ++q4)
          av[j][q4] = __builtin_amdgcn_raw_buffer_load_b128(acc_rsrc, (int)((part * 128 + 32 * g + 4 * q4) * 4), 0, 1 << 4);
      }
      float Mn = M;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (s0 + j < p.n_split) Mn = fmaxf(Mn, ms[j]);
      if (Mn != kNegInf) {
        const float keep = (M == kNegInf) ? 0.f : fast_exp2(M - Mn);
#pragma unroll
        for (int d = 0; d < 32; ++d) tot[d] *= keep;
        L *= keep;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float f = (s0 + j >= p.n_split || ms[j] == kNegInf) ? 0.f : fast_exp2(ms[j] - Mn);
#pragma unroll
          for (int q4 = 0; q4 < 8; ++q4) {
            tot[4 * q4 + 0] = fmaf(__uint_as_float(av[j][q4].x), f, tot[4 * q4 + 0]);
            tot[4 * q4 + 1] = fmaf(__uint_as_float(av[j][q4].y), f, tot[4 * q4 + 1]);
            tot[4 * q4 + 2] = fmaf(__uint_as_float(av[j][q4].z), f, tot[4 * q4 + 2]);
            tot[4 * q4 + 3] = fmaf(__uint_as_float(av[j][q4].w), f, tot[4 * q4 + 3]);
          }
          L = fmaf(ls[j], f, L);
        }
      }
      M = Mn;
    }
    char *dst = p.out + (r * p.o_sr + (int64_t)hq * p.o_sh + 32 * g) * 2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float o8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o8[e] = L > 0.f ? tot[8 * i + e] / L : 0.f;
      uint4 o;
      o.x = E::pack(o8[0], o8[1]);
      o.y = E::pack(o8[2], o8[3]);
      o.z = E::pack(o8[4], o8[5]);
      o.w = E::pack(o8[6], o8[7]);
      *reinterpret_cast<uint4 *>(dst + 16 * i) = o;
    }
    if (g == 0 && p.lse) p.lse[r * p.Hq + hq] = L > 0.f ? (M + log2f(L)) * kLn2 : kNegInf;
  }
}

// Fixed split: grid = (query rows, kv-head groups, splits); every row's chunks are cut into
// n_split equal runs. kMaxThreads bounds the workgroup size, which with one workgroup per CU fixes
// the register budget (256 threads: one wavefront per SIMD, 512 registers).
template <typename E, int kDepth, int kMaxThreads, bool kMergeHere = false>
__global__ __launch_bounds__(kMaxThreads, 1) void swa_decode_split_mfma_kernel(const DecodeParams p, const int G,
                                                                                const int Hkv) {
  const int64_t r = blockIdx.x;
  if (r >= p.rows) return;  // (the row count is padded to a multiple of 8 when the merge is done in here)
  const int split = blockIdx.z;
  const int tid = threadIdx.x;
  // (the row's length is asked for before anything else: it heads the chain length -> table -> K/V)
  int lo, hi, first_chunk;
  const int n_chunks = row_chunks(p, p.seq_lens, r, lo, hi, first_chunk);
  const int kvh = blockIdx.y * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(tid >> 6);
  if (kvh >= Hkv) return;  // whole wavefront; there is no barrier in this kernel
  const int cps = (n_chunks + p.n_split - 1) / p.n_split;
  const int cb = first_chunk + split * cps;
  const int ce = min(cb + cps, first_chunk + n_chunks);
  split_segment<E, kDepth, 1, kMergeHere>(p, p.block_table, G, kvh, tid & 63, r, lo, hi, cb, ce, ce == first_chunk + n_chunks,
                           p.n_split == 1, r * p.Hq * p.n_split + split, p.n_split,
                           split, p.meta_len > 0 ? p.n_split : 0);  // meta chunks dealt round robin to the splits
}

__device__ __forceinline__ int wave_sum(int x) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) x += __shfl_xor(x, d);
  return x;
}
__device__ __forceinline__ int wave_inclusive_scan(int x, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  return x;
}

// Balanced split: the chunks of all rows, laid end to end in row order, are cut into gridDim.x
// equal runs, one per workgroup, whatever the rows' lengths (a fixed split leaves the workgroups
// of short rows idle while the longest finish). A run may cover the end of one row, whole short
// rows and the start of another: one partial per (workgroup w, row r) it touches, stored as
// partial number w + r (both grow along the runs, so the sum is unique). Every wavefront works
// out the runs from seq_lens by itself: a few wave-wide sums, no communication. The tables are
// separate restrict-qualified parameters: the partial stores of one row come before the table
// lookups of the next, and only with the no-alias guarantee do those lookups stay scalar loads
// (as vector loads each would wait for every K/V load in flight).
template <typename E, int kDepth, int kMaxThreads>
__global__ __launch_bounds__(kMaxThreads, 1) void swa_decode_balanced_mfma_kernel(
    const DecodeParams p, const int32_t *__restrict__ block_table, const int32_t *__restrict__ seq_lens, const int G,
    const int Hkv) {
  const int tid = threadIdx.x;
  const int kvh = blockIdx.y * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(tid >> 6);
  if (kvh >= Hkv) return;
  const int lane = tid & 63;
  const int w = blockIdx.x, n_wg = gridDim.x;
  // Every wavefront works the runs out for itself from one look at seq_lens: lane i holds row base + i (its
  // visible range and chunks); a wave-wide scan places the rows on the common chunk axis; the rows of this
  // workgroup's run are then read back from those lanes (no second trip to memory per row).
  int total = 0;
  if (p.rows > 64) {  // more rows than lanes: the total needs a pass of its own
    for (int base = 0; base < p.rows; base += 64) {
      int lo, hi, fc;
      const int nn = base + lane < p.rows ? row_chunks(p, seq_lens, base + lane, lo, hi, fc) : 0;
      total += wave_sum(nn > 0 ? nn + kBalancedRowStartChunks : 0);
    }
    total = __builtin_amdgcn_readfirstlane(total);
  }
  int before = 0;  // chunks of the rows below `base`
  int per = 0, c0 = 0, c1 = 0;
  for (int base = 0; base < p.rows; base += 64) {
    int lo = 0, hi = 0, fc = 0;
    const int n = base + lane < p.rows ? row_chunks(p, seq_lens, base + lane, lo, hi, fc) : 0;
    const int len = n > 0 ? n + kBalancedRowStartChunks : 0;   // the row on the common axis: virtual chunks, then its own
    const int incl = wave_inclusive_scan(len, lane);
    if (base == 0) {
      if (p.rows <= 64) total = __builtin_amdgcn_readlane(incl, 63);
      per = (total + n_wg - 1) / n_wg;
      c0 = w * per;
      c1 = min(c0 + per, total);
      if (c0 >= c1) return;
    }
    if (before >= c1) break;
    const int start = before + incl - n;  // this lane's row's own chunks begin at this chunk of the whole
    uint64_t todo = __builtin_amdgcn_ballot_w64(n > 0 && start < c1 && start + n > c0);
    while (todo) {
      const int i = __builtin_ctzll(todo);
      todo &= todo - 1;
      const int r_start = __builtin_amdgcn_readlane(start, i);
      const int rlo = __builtin_amdgcn_readlane(lo, i), rhi = __builtin_amdgcn_readlane(hi, i);
      const int rfc = __builtin_amdgcn_readlane(fc, i), rn = __builtin_amdgcn_readlane(n, i);
      const int64_t r = base + i;
      const int cb = rfc + max(c0 - r_start, 0), ce = rfc + min(c1 - r_start, rn);
      split_segment<E, kDepth, 2>(p, block_table, G, kvh, lane, r, rlo, rhi, cb, ce, ce == rfc + rn, false,
                                  (int64_t)(w + r) * p.Hq, 1, 0, 0);
    }
    before += __builtin_amdgcn_readlane(incl, 63);
  }
}

}  // namespace

namespace sb_host {

// Launches the matrix-core split kernel (dtype bf16 or fp16, group size <= 16).
// `rows`, `n_split` give grid x and z; the kv heads are spread over wavefronts and grid y.
// With p.n_wg > 0 the balanced kernel runs instead: p.n_wg workgroups per kv-head group.
void launch_swa_decode_split_mfma(int dtype, int G, int Hkv, unsigned rows, unsigned n_split, int depth,
                                  hipStream_t st, const sb::DecodeParams &p, hipEvent_t ev_start, hipEvent_t ev_stop) {
  // up to 4 wavefronts (kv heads) per workgroup: one per SIMD, each with the whole register file
  const int waves = Hkv < 4 ? Hkv : 4;
  const unsigned ygroups = (unsigned)((Hkv + waves - 1) / waves);
  const dim3 block(64 * waves);
  // measured on the 7B decode shape: one chunk of prefetch is as fast as two or three
  if (depth <= 0) depth = 1;
  if (p.n_wg > 0) {
    const dim3 grid((unsigned)p.n_wg, ygroups);
    if (dtype == SB_BF16)
      hipLaunchKernelGGL((swa_decode_balanced_mfma_kernel<sb::BF16, 1, 256>), grid, block, 0, st, p, p.block_table,
                         p.seq_lens, G, Hkv);
    else
      hipLaunchKernelGGL((swa_decode_balanced_mfma_kernel<sb::F16, 1, 256>), grid, block, 0, st, p, p.block_table,
                         p.seq_lens, G, Hkv);
    return;
  }
  // merge inside this kernel: all splits of a row on one XCD (workgroup i runs on XCD i % 8, and the number of
  // a workgroup is x + gridDim.x * (y + gridDim.y * z)), which a row count padded to a multiple of 8 gives
  const dim3 grid(p.merge_counter ? (rows + 7u) / 8u * 8u : rows, ygroups, n_split);
  if (p.merge_counter) {  // the variant that merges the partial results itself (depth 1 only)
    if (dtype == SB_BF16)
      hipLaunchKernelGGL((swa_decode_split_mfma_kernel<sb::BF16, 1, 256, true>), grid, block, 0, st, p, G, Hkv);
    else
      hipLaunchKernelGGL((swa_decode_split_mfma_kernel<sb::F16, 1, 256, true>), grid, block, 0, st, p, G, Hkv);
    return;
  }
  if (ev_start && ev_stop && depth == 1) {  // timed launch: the events ride on the kernel's own dispatch
    if (dtype == SB_BF16)
      hipExtLaunchKernelGGL((swa_decode_split_mfma_kernel<sb::BF16, 1, 256>), grid, block, 0, st, ev_start, ev_stop, 0, p, G, Hkv);
    else
      hipExtLaunchKernelGGL((swa_decode_split_mfma_kernel<sb::F16, 1, 256>), grid, block, 0, st, ev_start, ev_stop, 0, p, G, Hkv);
    return;
  }
#define SB_LAUNCH(E, D) hipLaunchKernelGGL((swa_decode_split_mfma_kernel<E, D, 256>), grid, block, 0, st, p, G, Hkv)
  if (dtype == SB_BF16) {
    if (depth == 1) SB_LAUNCH(sb::BF16, 1);
    else if (depth == 2) SB_LAUNCH(sb::BF16, 2);
    else SB_LAUNCH(sb::BF16, 3);
  } else {
    if (depth == 1) SB_LAUNCH(sb::F16, 1);
    else if (depth == 2) SB_LAUNCH(sb::F16, 2);
    else SB_LAUNCH(sb::F16, 3);
  }
#undef SB_LAUNCH
}

}  // namespace sb_host
