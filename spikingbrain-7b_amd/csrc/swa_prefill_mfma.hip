// Causal sliding-window attention for many query tokens per sequence (prefill, chunked prefill,
// multi-token decode), bf16/fp16, on the matrix cores. Keys/values come either from the step's own
// key/value tensors (plain prompt) or from the paged cache through the block table (chunked prefill,
// prefix reuse). Replaces the varlen flash-attention call of
// vllm_hymeta/attention/fa_kernel_metatoken.py:235-253 (window_size=(window_left, 0), causal aligned to
// the end of the key sequence).
//
// Work decomposition
//   grid = (query tiles of 64 tokens, kv heads); a workgroup covers up to 4 query heads of the kv head
//   (a wider GQA group takes several launches, 7 = 4 + 3). Every wavefront owns two "column blocks" of
//   16 tokens x 1 head (32 score columns, no padding): a pair of heads is served by 4 wavefronts (one
//   per 16-token sub-tile), an odd last head by 2 wavefronts (two sub-tiles each) - 8 wavefronts for 4
//   heads, 6 for 3. At 256 registers per wavefront two of them share a SIMD.
//   The workgroup walks the union of its tokens' windows in chunks of 32 keys. Each chunk of K and V
//   (32 rows x 256 B each) is fetched from global memory ONCE per workgroup (every wavefront of an
//   8-wavefront workgroup fetches 4 rows with whole-row 16-byte lanes, else the first four fetch 8) into a
//   ring of three LDS chunks whose rows are padded to 288 B; all wavefronts then read their MFMA operands
//   from LDS. Global loads run three chunks ahead of the arithmetic (two register sets used alternately, the
//   loop written out for both). They are ordinary cached loads: the neighbouring query tiles, which run at
//   the same time on the same XCD, read the same rows. The arithmetic is staggered over two chunks: an
//   iteration issues the scores of chunk x+1 ahead of the numerators of chunk x, and the P V product of
//   chunk x ahead of the masking and maxima of chunk x+1, so that a wavefront's matrix instructions have
//   vector work of another chunk behind them.
//   A wavefront issues about one instruction per 5 cycles whatever its kind, and a scalar branch costs 15-25
//   cycles, so the loop is kept short: everything that does not depend on the lane lives in scalar registers
//   (a chunk's address is one block-table entry, read one iteration ahead, times the block stride, plus the
//   K and V bases; a lane adds a 32-bit offset), the range of chunks that need no masking is computed once,
//   and the rare paths (masking, raising the reference point) sit behind one branch each.
//   Meta rows, when given, are taken in a loop of their own in front of the walk.
//   Per chunk and column block: S^T = K Q^T (8 MFMA 16x16x32, tokens on the N axis), softmax numerators
//   per lane for token lane%16 in log2 units, O^T += V^T P^T (8 MFMA). P stays in the lane that produced
//   it; V^T operands come out of the [key][dim] stage through the transposing LDS load, shared by the two
//   blocks.
//   Workgroups are numbered so that each XCD (own L2) works through one contiguous run of tiles.
//
// Softmax reference point
//   The numerators are exp2(s - m_ref) with a per-row reference m_ref that is only raised when some
//   row of the wavefront scores more than kRaise (log2 units) above it, so they stay below 2^kRaise
//   (exact in fp32 sums, inside fp16 range). The check uses each lane's own 8 keys, so the common case
//   has no cross-lane traffic; raising m_ref (rare after the first chunks) takes the row maximum over
//   the four lanes of a token and rescales the output accumulators.
#include "common.h"
#include "mfma_util.h"

namespace {

using namespace sb;

struct PrefillParams {
  const char *q;
  const char *k;
  const char *v;
  char *out;
  float *lse;                 // [total_q, Hq] natural-log log-sum-exp, or null
  // byte-code caches (paged): per-row INT8 scales [nb, Hkv, bs], or one fp8 scale per tensor
  const float *k_scale;
  const float *v_scale;
  float k_scale_tensor, v_scale_tensor;
  int Hkv;
  const int32_t *block_table;
  const int64_t *kv_start;
  const int32_t *key_lo;      // [S] first visible key of each sequence, or null
  const int32_t *cu_q;        // [S+1] first q/out row of each sequence
  const int32_t *seq_lens_k;  // [S] keys of each sequence (context + new tokens)
  const int32_t *tile_seq;    // [tiles] sequence of each 64-token query tile
  const int32_t *tile_q0;     // [tiles] first query (index inside its sequence) of the tile
  int G, head_begin;          // query heads per kv head; first of them handled by this launch
  int Hq;
  int num_tiles;
  int block_size, window_left;
  int tiles_per_block;        // block_size / 16
  uint32_t tpb_magic;         // ceil(2^31 / tiles_per_block): tile -> block by one multiplication
  float scale_log2;
  int64_t q_sr, q_sh, o_sr, o_sh;  // elements
  int64_t kv_sb, kv_sr, kv_sh;     // bytes
  int64_t bt_stride;
  // Meta tokens: meta_len rows [meta_len, Hkv, 128] of the query's type every query also attends to,
  // unmasked, in the same softmax: they are walked as the chunks in front of the window's. 0 = none.
  const char *meta_k;
  const char *meta_v;
  int meta_len;
  int64_t meta_sr, meta_sh;  // bytes
  ScoreOptions opt;          // soft cap / ALiBi slopes, applied to every raw score in front of the mask
  // ALiBi term of meta row j for packed query row t: -slope * |meta_bias_off + t - j|, meta_bias_off = row0 + meta_len - rows
  int meta_bias_off;
};

#ifndef SB_PREFILL_HEADS
#define SB_PREFILL_HEADS 4
#endif
constexpr int kRowPad = 288;   // LDS row stride of a K chunk: 256 B of data + 32 B (16-byte operand loads of 16 rows: measured 1.6 x the rate of a 272 B stride)
constexpr int kRowPadV = 288;  // of a V chunk: 256 B + 32 B (transposing loads: 4 rows x 32 B at a time)
constexpr int kStageK = 32 * kRowPad, kStageV = 32 * kRowPadV;
constexpr int kStage = kStageK + kStageV;  // one chunk of K and V

// ds_read_b64_tr_b16: in every group of 16 lanes, lane i names 8 bytes (4 elements) of LDS, "row i"; lane l
// receives element l % 4 of rows l / 4, l / 4 + 4, l / 4 + 8, l / 4 + 12. With row i = (key k0 + i / 4, dims
// d0 + 4 (i % 4) .. + 3), lane l gets dim d0 + l of keys k0 .. k0 + 3: V^T straight out of a [key][dim] stage.
__device__ __forceinline__ uint2 load_transposed(const char *row) {
  typedef short v4s __attribute__((ext_vector_type(4)));
  const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)row);
  return __builtin_bit_cast(uint2, v);
}
constexpr float kNegInf = kNegInfF;
constexpr float kRaise = 8.f;

// NHEADS query heads of one kv head per workgroup; wavefronts own two column blocks each
// (a column block = 16 tokens x 1 head): head pairs are served by 4 wavefronts (one per 16-token
// sub-tile, both heads of the pair), an odd last head by 2 wavefronts (two sub-tiles each).
template <int NHEADS>
struct Shape {
  static constexpr int kPairs = NHEADS / 2;
  static constexpr int kWaves = 4 * kPairs + 4 * (NHEADS % 2);
  static constexpr int kFetchWaves = kWaves == 8 ? 8 : (kWaves < 4 ? kWaves : 4);   // wavefronts that move K/V into LDS
  static constexpr int kLoads = 8 / kFetchWaves;                // 4-row loads per fetching lane, per K and per V
};

// The registers a fetching lane carries a chunk in: 16-byte pieces of K and V rows, or, for a byte-code
// cache (KVQ = SB_KV_INT8 / SB_KV_FP8), the 8 codes that become such a piece plus (INT8) their row's scales.
template <int KVQ, int N>
struct StageSet {
  uint4 k[N], v[N];
};
template <int N>
struct StageSet<SB_KV_INT8, N> {
  uint2 k[N], v[N];
  float ks[N], vs[N];
};
template <int N>
struct StageSet<SB_KV_FP8, N> {
  uint2 k[N], v[N];
};

template <int Q, int B>
__device__ __forceinline__ float code_value(uint32_t w) {
  if constexpr (Q == SB_KV_INT8) return (float)(int)(int8_t)(w >> (8 * B));
  else return __builtin_amdgcn_cvt_f32_fp8((int)w, B);
}
// 8 codes times their scale, rounded to E: the values the reference attends to after its own
// quantise-dequantise (code * scale cast back to the tensor's dtype)
template <typename E, int Q>
__device__ __forceinline__ uint4 dequant8(uint2 w, float s) {
  return make_uint4(Mma<E>::pack(code_value<Q, 0>(w.x) * s, code_value<Q, 1>(w.x) * s),
                    Mma<E>::pack(code_value<Q, 2>(w.x) * s, code_value<Q, 3>(w.x) * s),
                    Mma<E>::pack(code_value<Q, 0>(w.y) * s, code_value<Q, 1>(w.y) * s),
                    Mma<E>::pack(code_value<Q, 2>(w.y) * s, code_value<Q, 3>(w.y) * s));
}

template <typename E, int NHEADS, int KVQ, bool PAGED>
__global__ __attribute__((amdgpu_flat_work_group_size(64 * Shape<NHEADS>::kWaves, 64 * Shape<NHEADS>::kWaves),
                          amdgpu_waves_per_eu(2, 2)))
void swa_prefill_kernel(const PrefillParams p) {
  using S = Shape<NHEADS>;
  __shared__ __attribute__((aligned(16))) char smem[3 * kStage];  // ring of three chunks, each [K|V]

  // Workgroups are handed to the 8 XCDs round-robin by index, and each XCD has its own L2. Give XCD x
  // the x-th contiguous eighth of the tiles, so that the workgroups resident on one XCD at a time are
  // neighbouring tiles of one sequence and kv head, whose key windows overlap almost entirely.
  const int per_xcd = (p.num_tiles + 7) >> 3;
  const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (tile >= p.num_tiles) return;
  const int kvh = blockIdx.y;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int g = lane >> 4;
  const int c = lane & 15;

  const int seq = p.tile_seq[tile];
  const int q0 = p.tile_q0[tile];
  const int qrow0 = p.cu_q[seq];
  const int Lq = p.cu_q[seq + 1] - qrow0;
  const int Lk = p.seq_lens_k[seq];
  const int shift = Lk - Lq;  // query j sits at key index shift + j
  const int wl = p.window_left;

  // keys any token of this workgroup can see: [wg_lo, wg_hi)
  const int j_last = min(q0 + 63, Lq - 1);
  const int wg_hi = shift + j_last + 1;
  const int klo = p.key_lo ? max(p.key_lo[seq], 0) : 0;
  // (kept inside the sequence even when padding hides every key: such rows end up fully masked)
  const int wg_lo = min(max(wl >= 0 ? shift + q0 - wl : 0, klo), wg_hi - 1);
  const int first_tile = wg_lo >> 4, last_tile = (wg_hi - 1) >> 4;
  const int ch_begin = wg_lo >> 5, ch_end = ((wg_hi - 1) >> 5) + 1;
  const int n_walk = ch_end - ch_begin;  // the walk: index x is window chunk ch_begin + x
  const int meta_chunks = (p.meta_len + 31) >> 5;

  // Everything from here on is written for NB column blocks per wavefront: two for the wavefronts of a head
  // pair, one for those of an odd last head (four wavefronts, one per 16-token sub-tile).
  auto run = [&](auto nb_tag) __attribute__((always_inline)) {
    constexpr int NB = decltype(nb_tag)::value;
    // this wavefront's NB column blocks: 16-token sub-tile ts[b] of head hd[b]
    int ts[NB], hd[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      ts[b] = wave & 3;
      hd[b] = NB == 2 ? 2 * (wave >> 2) + b : NHEADS - 1;
    }
    const int head0 = kvh * p.G + p.head_begin;
    // (rows past the end of the sequence repeat its last token; they are never stored)
    const int jw0 = min(q0 + 16 * ts[0], Lq - 1);            // first and last token of the wavefront
    const int jw_last = min(q0 + 16 * ts[NB - 1] + 15, Lq - 1);
    int my_pos[NB], my_lo[NB];
    uint4 qb[NB][4];  // Q^T operands: token lane%16 of the block, dims of 16-byte piece 4s+g
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int j_mine = min(q0 + 16 * ts[b] + c, Lq - 1);
      my_pos[b] = shift + j_mine;
      my_lo[b] = max(wl >= 0 ? my_pos[b] - wl : 0, klo);
#pragma unroll
      for (int s = 0; s < 4; ++s)
        qb[b][s] = *reinterpret_cast<const uint4 *>(
            p.q + ((int64_t)(qrow0 + j_mine) * p.q_sr + (int64_t)(head0 + hd[b]) * p.q_sh + (4 * s + g) * 8) * 2);
    }
    // Chunks wholly visible to every token of the wavefront (at or above every token's lower bound, at or below
    // the first token) need no masking: walk indices [full_lo, full_lo + full_cnt).
    const int vis_lo = max(wl >= 0 ? shift + jw_last - wl : 0, klo);
    const int full_lo = ((vis_lo + 31) >> 5) - ch_begin;
    const unsigned full_cnt = (unsigned)max(((shift + jw0 + 1) >> 5) - ch_begin - full_lo, 0);

    f32x4_t acc[NB][8];
    float m[NB], l[NB];  // m: reference point of the numerators (log2 units), l: this lane's share of the sum
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      m[b] = kNegInf;
      l[b] = 0.f;
#pragma unroll
      for (int mt = 0; mt < 8; ++mt) acc[b][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // ---- global -> registers -> LDS: the first kFetchWaves wavefronts move the chunk (32 K rows and
    // 32 V rows of 256 B); each of their loads covers 4 rows, all inside one 16-key tile of the table.
    // Rows outside [wg_lo, wg_hi) are clamped onto the nearest visible key (masked for every token).
    // Everything that does not depend on the lane is kept in scalar registers: per chunk, the tile's byte offset
    // (one block-table entry, looked up one call ahead of its use) added to the K and V bases; a lane adds its
    // row and column as a 32-bit offset.
    constexpr int kFetchAll = S::kFetchWaves == S::kWaves;
    const bool fetcher = kFetchAll || wave < S::kFetchWaves;
    constexpr int rows_per_wave = 32 / S::kFetchWaves;                     // 4, 8 or 16
    const int tsel = (wave * rows_per_wave) >> 4;                          // which 16-key tile of a chunk this wavefront's rows are in
    const int lrow = (wave * rows_per_wave) % 16 + (lane >> 4);            // row inside the tile, +4 per load
    const uint32_t row_bytes = (uint32_t)p.kv_sr;                          // < 2^24 (host check)
    const uint32_t lane_col = c * (KVQ == SB_KV_NONE ? 16 : 8);
    const int64_t wg_off = (int64_t)kvh * p.kv_sh + ((!PAGED && p.kv_start) ? p.kv_start[seq] * p.kv_sr : 0);
    const char *const kbase = p.k + wg_off, *const vbase = p.v + wg_off;
    const int32_t *const table_row = PAGED ? p.block_table + (int64_t)seq * p.bt_stride : nullptr;
    auto walk_tile = [&](int x) __attribute__((always_inline)) {  // (past the end of the walk: the last tile again)
      return min(max(2 * (ch_begin + x) + tsel, first_tile), last_tile);
    };
    // block of 16-key tile t: t / tiles_per_block by multiplication (exact while t < 2^31 / tiles_per_block)
    auto block_of = [&](int t) __attribute__((always_inline)) { return (int)__umulhi((uint32_t)t << 1, p.tpb_magic); };
    int next_blk = 0;  // table entry of the tile the next fetch takes
    if constexpr (PAGED) next_blk = table_row[block_of(walk_tile(0))];
    int fx = 0;        // walk index the next fetch takes
    using Set = StageSet<KVQ, S::kLoads>;
    Set stage[2];  // walk index x travels in set x & 1
    auto fetch = [&](Set &st) __attribute__((always_inline)) {
      const int t = walk_tile(fx);
      ++fx;
      int64_t off;  // of the tile's first row from kbase / vbase
      [[maybe_unused]] int64_t scale_row = 0;  // INT8: index of that row in the scale tensors
      if constexpr (PAGED) {
        const int bi = block_of(t);
        const int64_t blk = next_blk;
        next_blk = table_row[block_of(walk_tile(fx))];
        const int in_block = (t - bi * p.tiles_per_block) << 4;
        off = blk * p.kv_sb + (int64_t)((uint32_t)in_block * row_bytes);
        if constexpr (KVQ == SB_KV_INT8) scale_row = (blk * p.Hkv + kvh) * p.block_size + in_block;
      } else {
        off = (int64_t)(t << 4) * p.kv_sr;
      }
      const char *const kp = kbase + off, *const vp = vbase + off;
      const int lo = wg_lo - (t << 4), hi = wg_hi - 1 - (t << 4);
#pragma unroll
      for (int u = 0; u < S::kLoads; ++u) {
        const int row = min(max(lrow + 4 * u, lo), hi);  // inside the tile: 0 .. 15
        const uint32_t vo = __umul24((uint32_t)row, row_bytes) + lane_col;
        if constexpr (KVQ == SB_KV_NONE) {
          st.k[u] = *reinterpret_cast<const uint4 *>(kp + vo);  // (cached: the neighbouring query tiles read the same rows)
          st.v[u] = *reinterpret_cast<const uint4 *>(vp + vo);
        } else {  // a row is 128 code bytes: 8 per lane
          const unsigned long long wk = *reinterpret_cast<const unsigned long long *>(kp + vo);
          const unsigned long long wv = *reinterpret_cast<const unsigned long long *>(vp + vo);
          st.k[u] = make_uint2((uint32_t)wk, (uint32_t)(wk >> 32));
          st.v[u] = make_uint2((uint32_t)wv, (uint32_t)(wv >> 32));
          if constexpr (KVQ == SB_KV_INT8) {
            st.ks[u] = (p.k_scale + scale_row)[(uint32_t)row];
            st.vs[u] = (p.v_scale + scale_row)[(uint32_t)row];
          }
        }
      }
    };
    const int stash_off = (wave * rows_per_wave + (lane >> 4)) * kRowPad + c * 16;   // of this lane's first row in a K chunk;
    const int stash_off_v = (wave * rows_per_wave + (lane >> 4)) * kRowPadV + c * 16 + kStageK;  // in the V chunk behind it
    auto stash = [&](int slot, const Set &st) __attribute__((always_inline)) {  // slot = byte offset of a ring slot
      char *sk = smem + slot + stash_off, *sv = smem + slot + stash_off_v;
#pragma unroll
      for (int u = 0; u < S::kLoads; ++u) {
        uint4 kq, vq;
        if constexpr (KVQ == SB_KV_NONE) {
          kq = st.k[u];
          vq = st.v[u];
        } else if constexpr (KVQ == SB_KV_INT8) {
          kq = dequant8<E, KVQ>(st.k[u], st.ks[u]);
          vq = dequant8<E, KVQ>(st.v[u], st.vs[u]);
        } else {
          kq = dequant8<E, KVQ>(st.k[u], p.k_scale_tensor);
          vq = dequant8<E, KVQ>(st.v[u], p.v_scale_tensor);
        }
        *reinterpret_cast<uint4 *>(sk + 4 * u * kRowPad) = kq;
        *reinterpret_cast<uint4 *>(sv + 4 * u * kRowPadV) = vq;
      }
    };

    // Scores live in two register sets used alternately: while the numerators of one chunk are formed in one set,
    // the matrix instructions write the next chunk's scores into the other. s[b][t][i]: block b, key 16 t + 4 g + i
    // of the chunk (raw dot products; -inf where masked).
    using Scores = f32x4_t[NB][2];
    Scores sa, sb2;
    float mx[NB];    // row maxima of the scores whose softmax comes next, in log2 units
    uint4 pb[NB];    // probabilities of the chunk whose P V product comes next

    // The two halves of an iteration. Each runs 16 matrix instructions next to the vector work of another chunk
    // that does not depend on them.
    //
    // first half: S^T = K Q^T of the next chunk (kNext; K from ring slot `slot`) into `sn`, next to the
    // numerators of the chunk in `sc` against the current reference points (kCur) -> pb, l.
    auto first_half = [&](int slot, Scores &sn, Scores &sc, auto next_tag, auto cur_tag) __attribute__((always_inline)) {
      constexpr bool kNext = decltype(next_tag)::value, kCur = decltype(cur_tag)::value;
      const char *sk0 = smem + slot + c * kRowPad + g * 16, *sk1 = sk0 + 16 * kRowPad;
      uint4 k0[4], k1[4];  // operand loads run one step ahead of their use (two pairs live)
      if constexpr (kNext) {
        k0[0] = *reinterpret_cast<const uint4 *>(sk0);
        k1[0] = *reinterpret_cast<const uint4 *>(sk1);
#pragma unroll
        for (int b = 0; b < NB; ++b) sn[b][0] = sn[b][1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      }
      float m_safe[NB], psum[NB];
#pragma unroll
      for (int b = 0; b < NB; ++b) m_safe[b] = (m[b] == kNegInf) ? 0.f : m[b];
      if constexpr (kNext) {  // 2 NB chains (block, tile), each four instructions deep, taken in turn
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          if (s + 1 < 4) {
            k0[s + 1] = *reinterpret_cast<const uint4 *>(sk0 + (s + 1) * 64);
            k1[s + 1] = *reinterpret_cast<const uint4 *>(sk1 + (s + 1) * 64);
          }
#pragma unroll
          for (int b = 0; b < NB; ++b) {
            sn[b][0] = Mma<E>::run(k0[s], qb[b][s], sn[b][0]);
            sn[b][1] = Mma<E>::run(k1[s], qb[b][s], sn[b][1]);
          }
        }
      }
      if constexpr (kCur) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          psum[b] = 0.f;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float e = fast_exp2(fmaf(sc[b][j >> 2][j & 3], p.scale_log2, -m_safe[b]));
            sc[b][j >> 2][j & 3] = e;
            psum[b] += e;
          }
        }
      }
      if constexpr (kCur) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          l[b] += psum[b];
          pb[b] = make_uint4(Mma<E>::pack(sc[b][0][0], sc[b][0][1]), Mma<E>::pack(sc[b][0][2], sc[b][0][3]),
                             Mma<E>::pack(sc[b][1][0], sc[b][1][1]), Mma<E>::pack(sc[b][1][2], sc[b][1][3]));
        }
      }
    };

    // second half: O^T += V^T P^T (kPV; probabilities pb), next to the row maxima of the (masked) scores `sn` of
    // the next chunk (kPost). True when some row of that chunk needs a higher reference point.
    // V^T operands of a chunk, dims 16 mt + c: this lane's 8 keys (4g .. 4g+3 of either 16-key tile, the order of
    // its probabilities) by two transposing loads per mt; built once, used by both blocks. They are requested at
    // the top of an iteration and arrive while the first half runs.
    uint2 vlo[8], vhi[8];
    auto load_v = [&](int slot) __attribute__((always_inline)) {
      const char *v0 = smem + slot + kStageK + (4 * g + (c >> 2)) * kRowPadV + (c & 3) * 8, *v1 = v0 + 16 * kRowPadV;
#pragma unroll
      for (int mt = 0; mt < 8; ++mt) {
        vlo[mt] = load_transposed(v0 + mt * 32);
        vhi[mt] = load_transposed(v1 + mt * 32);
      }
    };
    auto second_half = [&](const Scores &sn, auto pv_tag, auto post_tag) __attribute__((always_inline)) -> bool {
      constexpr bool kPV = decltype(pv_tag)::value, kPost = decltype(post_tag)::value;
      float t[NB];
      if constexpr (kPV) {
#pragma unroll
        for (int mt = 0; mt < 8; ++mt)
#pragma unroll
          for (int b = 0; b < NB; ++b)
            acc[b][mt] = Mma<E>::run(make_uint4(vlo[mt].x, vlo[mt].y, vhi[mt].x, vhi[mt].y), pb[b], acc[b][mt]);
      }
      if constexpr (kPost) {  // each lane checks its own 8 keys: no cross-lane traffic unless the reference point must move
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          t[b] = kNegInf;
#pragma unroll
          for (int j = 0; j < 8; ++j) t[b] = fmaxf(t[b], sn[b][j >> 2][j & 3]);
        }
      }
      bool raise = false;
      if constexpr (kPost) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          mx[b] = t[b] * p.scale_log2;
          raise |= mx[b] > m[b] + kRaise;  // also true for the first finite score of a row (m = -inf)
        }
      }
      return __builtin_amdgcn_ballot_w64(raise) != 0;
    };
    // Soft cap / ALiBi on the scores of walk index xn, in place (only when asked for: one uniform branch).
    float my_slope[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) my_slope[b] = p.opt.slopes ? p.opt.slopes[head0 + hd[b]] : 0.f;
    auto adjust_scores = [&](int xn, Scores &sn) __attribute__((always_inline)) {
      if (!p.opt.on) return;
      const int c0 = (ch_begin + xn) << 5;
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          sn[b][j >> 2][j & 3] = adjust_score(p.opt, sn[b][j >> 2][j & 3], my_slope[b],
                                              (float)(c0 + ((j >> 2) << 4) + 4 * g + (j & 3) - my_pos[b]));
    };
    // Masking of the scores of walk index xn, in place (selects, not branches: the comparison results are
    // combined as bits). Skipped for the chunks every token of the wavefront sees whole.
    auto mask_scores = [&](int xn, Scores &sn) __attribute__((always_inline)) {
      if ((unsigned)(xn - full_lo) < full_cnt) return;
      const int c0 = (ch_begin + xn) << 5;
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = c0 + ((j >> 2) << 4) + 4 * g + (j & 3);
          sn[b][j >> 2][j & 3] = bool((key > my_pos[b]) | (key < my_lo[b])) ? kNegInf : sn[b][j >> 2][j & 3];
        }
    };
    const std::true_type kYes{};
    const std::false_type kNo{};

    // lift the reference points to the running maxima and rescale what has been accumulated
    auto rescale = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        float t = mx[b];  // row maximum over the four lanes that share a token
        t = fmaxf(t, __shfl_xor(t, 16));
        t = fmaxf(t, __shfl_xor(t, 32));
        const float m_new = fmaxf(m[b], t);
        const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
        const float alpha = fast_exp2(m[b] - m_safe);
        m[b] = m_new;
        l[b] *= alpha;
#pragma unroll
        for (int mt = 0; mt < 8; ++mt) acc[b][mt] *= alpha;
      }
    };

    if (fetcher) {
      fetch(stage[0]);
      fetch(stage[1]);
    }
    // ---- meta rows: global -> ring slot 0 -> scores, one chunk at a time, while the first two chunks of the
    // window are on their way (every row that exists is visible to every token)
    for (int mc = 0; mc < meta_chunks; ++mc) {
      if (fetcher) {
        const char *mk = p.meta_k + (int64_t)kvh * p.meta_sh + c * 16, *mv = p.meta_v + (int64_t)kvh * p.meta_sh + c * 16;
#pragma unroll
        for (int u = 0; u < S::kLoads; ++u) {
          const int kk = wave * rows_per_wave + (lane >> 4) + 4 * u;
          const int64_t row = min((mc << 5) + kk, p.meta_len - 1);
          *reinterpret_cast<uint4 *>(smem + kk * kRowPad + c * 16) = *reinterpret_cast<const uint4 *>(mk + row * p.meta_sr);
          *reinterpret_cast<uint4 *>(smem + kStageK + kk * kRowPadV + c * 16) =
              *reinterpret_cast<const uint4 *>(mv + row * p.meta_sr);
        }
      }
      __syncthreads();
      first_half(0, sa, sa, kYes, kNo);
      if (p.opt.on) {  // soft cap / ALiBi on the meta rows: the distance of the reference's stacked second attention
        const int c0 = mc << 5;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          const int me = p.meta_bias_off + qrow0 + min(q0 + 16 * ts[b] + c, Lq - 1);
#pragma unroll
          for (int j = 0; j < 8; ++j)
            sa[b][j >> 2][j & 3] = adjust_score(p.opt, sa[b][j >> 2][j & 3], my_slope[b],
                                                -fabsf((float)(me - (c0 + ((j >> 2) << 4) + 4 * g + (j & 3)))));
        }
      }
      {
        const int c0 = mc << 5;
        float t[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          t[b] = kNegInf;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int key = c0 + ((j >> 2) << 4) + 4 * g + (j & 3);
            sa[b][j >> 2][j & 3] = key >= p.meta_len ? kNegInf : sa[b][j >> 2][j & 3];
            t[b] = fmaxf(t[b], sa[b][j >> 2][j & 3]);
          }
        }
        bool raise = false;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          mx[b] = t[b] * p.scale_log2;
          raise |= mx[b] > m[b] + kRaise;
        }
        if (__builtin_amdgcn_ballot_w64(raise) != 0) rescale();
      }
      first_half(0, sa, sa, kNo, kYes);
      load_v(0);
      second_half(sa, kYes, kNo);
      __syncthreads();
    }

    // ---- chunk loop: one barrier per chunk, every wavefront visits every chunk -------------------
    // (chunks outside a wavefront's own band come out fully masked and add zero)
    // Iteration x: scores of chunk x+1 while the numerators of chunk x are formed, then P V of chunk x while the
    // scores of chunk x+1 are masked and searched for their maxima; chunk x+2 goes from registers into the ring
    // slot that chunk x-1 has left, and chunk x+3 is requested from global memory into the registers chunk x+1
    // has left (two register sets and two score sets used alternately; the loop is written out for both so that
    // every register index is static). Loads are issued unconditionally (past the end they re-read the last
    // rows), so the wait in front of each LDS store counts exactly the loads that may still be in flight.
    int r0 = 0, r1 = kStage, r2 = 2 * kStage;  // ring slots of chunks x, x+1, x+2
    auto body = [&](int x, Scores &sc, Scores &sn, Set &arriving, Set &leaving) __attribute__((always_inline)) {
      load_v(r0);
      if (fetcher) fetch(arriving);  // chunk x + 3
      first_half(r1, sn, sc, kYes, kYes);
      adjust_scores(x + 1, sn);
      mask_scores(x + 1, sn);
      if (second_half(sn, kYes, kYes)) rescale();
      if (fetcher) stash(r2, leaving);  // chunk x + 2
      __syncthreads();
      const int t = r0;
      r0 = r1;
      r1 = r2;
      r2 = t;
    };
    if (fetcher) {
      stash(r0, stage[0]);
      fetch(stage[0]);  // chunk 2
      stash(r1, stage[1]);
    }
    __syncthreads();
    first_half(r0, sa, sa, kYes, kNo);
    adjust_scores(0, sa);
    mask_scores(0, sa);
    if (second_half(sa, kNo, kYes)) rescale();
    int x = 0;
    for (; x + 2 < n_walk; x += 2) {
      body(x, sa, sb2, stage[1], stage[0]);
      body(x + 1, sb2, sa, stage[0], stage[1]);
    }
    if (x + 1 < n_walk) {
      body(x, sa, sb2, stage[1], stage[0]);
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        sa[b][0] = sb2[b][0];
        sa[b][1] = sb2[b][1];
      }
    }
    // the last chunk: its numerators and its P V product
    load_v(r0);
    first_half(r1, sa, sa, kNo, kYes);
    second_half(sa, kYes, kNo);

    // ---- epilogue: lane (g, c) owns token c of each block, dims 16 mt + 4g + i --------------------------
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      float lt = l[b];
      lt += __shfl_xor(lt, 16);
      lt += __shfl_xor(lt, 32);
      if (q0 + 16 * ts[b] + c < Lq) {
        const float inv = lt > 0.f ? 1.f / lt : 0.f;
        char *dst = p.out + ((int64_t)(qrow0 + q0 + 16 * ts[b] + c) * p.o_sr + (int64_t)(head0 + hd[b]) * p.o_sh +
                             4 * g) * 2;
#pragma unroll
        for (int mt = 0; mt < 8; ++mt)
          *reinterpret_cast<uint2 *>(dst + 32 * mt) = make_uint2(E::pack(acc[b][mt][0] * inv, acc[b][mt][1] * inv),
                                                                 E::pack(acc[b][mt][2] * inv, acc[b][mt][3] * inv));
        if (p.lse && g == 0)
          p.lse[(int64_t)(qrow0 + q0 + 16 * ts[b] + c) * p.Hq + head0 + hd[b]] =
              lt > 0.f ? (m[b] + log2f(lt)) * kLn2 : kNegInf;
      }
    }
  };
  if constexpr (NHEADS % 2 == 1) {
    if (wave >= 4 * S::kPairs) run(std::integral_constant<int, 1>{});
    else if constexpr (NHEADS > 1) run(std::integral_constant<int, 2>{});
  } else {
    run(std::integral_constant<int, 2>{});
  }
}

template <typename E, int KVQ, bool PAGED>
void launch_prefill_q(int nh, dim3 grid, hipStream_t st, const PrefillParams &p) {
  switch (nh) {
    case 1: hipLaunchKernelGGL((swa_prefill_kernel<E, 1, KVQ, PAGED>), grid, dim3(64 * Shape<1>::kWaves), 0, st, p); break;
    case 2: hipLaunchKernelGGL((swa_prefill_kernel<E, 2, KVQ, PAGED>), grid, dim3(64 * Shape<2>::kWaves), 0, st, p); break;
    case 3: hipLaunchKernelGGL((swa_prefill_kernel<E, 3, KVQ, PAGED>), grid, dim3(64 * Shape<3>::kWaves), 0, st, p); break;
    default: hipLaunchKernelGGL((swa_prefill_kernel<E, 4, KVQ, PAGED>), grid, dim3(64 * Shape<4>::kWaves), 0, st, p); break;
  }
}
template <typename E>
void launch_prefill(int kv_quant, int nh, dim3 grid, hipStream_t st, const PrefillParams &p) {
  if (kv_quant == SB_KV_INT8) launch_prefill_q<E, SB_KV_INT8, true>(nh, grid, st, p);
  else if (kv_quant == SB_KV_FP8) launch_prefill_q<E, SB_KV_FP8, true>(nh, grid, st, p);
  else if (p.block_table) launch_prefill_q<E, SB_KV_NONE, true>(nh, grid, st, p);
  else launch_prefill_q<E, SB_KV_NONE, false>(nh, grid, st, p);
}

}  // namespace

extern "C" int sb_swa_prefill(const sb_swa_prefill_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_swa_prefill: null args");
  if (a->num_tiles < 0) return fail(SB_ERR_INVALID, "sb_swa_prefill: negative num_tiles");
  if (a->num_tiles == 0) return SB_OK;
  if (!a->q || !a->k || !a->v || !a->out || !a->cu_seqlens_q || !a->seq_lens_k || !a->tile_seq || !a->tile_q0)
    return fail(SB_ERR_INVALID, "sb_swa_prefill: null tensor pointer");
  if (a->head_size != 128)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_prefill: head_size %d (only 128 is built)", a->head_size);
  if (a->dtype != SB_BF16 && a->dtype != SB_F16)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_prefill: dtype must be bf16 or fp16");
  if (a->num_q_heads <= 0 || a->num_kv_heads <= 0 || a->num_q_heads % a->num_kv_heads != 0)
    return fail(SB_ERR_INVALID, "sb_swa_prefill: num_q_heads must be a positive multiple of num_kv_heads");
  if (!(a->scale > 0.f)) return fail(SB_ERR_INVALID, "sb_swa_prefill: scale must be positive");
  if (a->block_table && (a->block_size < 16 || a->block_size % 16 != 0))
    return fail(SB_ERR_INVALID, "sb_swa_prefill: block_size %d must be a multiple of 16", a->block_size);
  if (a->num_tiles > 0x7ffffff0LL || a->num_kv_heads > 65535)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_prefill: grid too large");
  const bool codes = a->kv_quant == SB_KV_INT8 || a->kv_quant == SB_KV_FP8;
  if (a->kv_quant != SB_KV_NONE && !codes)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_prefill: unknown kv_quant %d", a->kv_quant);
  if (codes && !a->block_table) return fail(SB_ERR_INVALID, "sb_swa_prefill: a byte-code cache needs paged mode");
  if (a->kv_quant == SB_KV_INT8 && (!a->k_scale || !a->v_scale))
    return fail(SB_ERR_INVALID, "sb_swa_prefill: the INT8 cache needs both scale tensors");
  if (a->kv_quant == SB_KV_FP8 && (!(a->k_scale_tensor > 0.f) || !(a->v_scale_tensor > 0.f)))
    return fail(SB_ERR_INVALID, "sb_swa_prefill: the fp8 cache needs positive k_scale_tensor and v_scale_tensor");
  const int kv_esz = codes ? 1 : 2;
  const int64_t es[] = {a->q_stride_row, a->q_stride_head, a->out_stride_row, a->out_stride_head};
  for (int64_t s : es)
    if ((s * 2) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_swa_prefill: stride %lld elements is not 16-byte aligned", (long long)s);
  const int64_t kes[] = {a->kv_stride_block, a->kv_stride_row, a->kv_stride_head};
  for (int64_t s : kes)
    if ((s * kv_esz) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_swa_prefill: cache stride %lld elements is not 16-byte aligned", (long long)s);
  if (a->kv_stride_row <= 0 || a->kv_stride_row * kv_esz >= (1 << 24))
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_prefill: cache row stride %lld elements (must be positive and below 16 MiB)",
                (long long)a->kv_stride_row);
  if ((reinterpret_cast<uintptr_t>(a->q) | reinterpret_cast<uintptr_t>(a->k) | reinterpret_cast<uintptr_t>(a->v) |
       reinterpret_cast<uintptr_t>(a->out)) & 15u)
    return fail(SB_ERR_INVALID, "sb_swa_prefill: q/k/v/out base not 16-byte aligned");

  PrefillParams p;
  p.q = (const char *)a->q; p.k = (const char *)a->k; p.v = (const char *)a->v; p.out = (char *)a->out;
  p.lse = a->lse; p.Hq = a->num_q_heads;
  p.block_table = a->block_table; p.kv_start = a->kv_start; p.key_lo = a->key_lo;
  p.cu_q = a->cu_seqlens_q; p.seq_lens_k = a->seq_lens_k; p.tile_seq = a->tile_seq; p.tile_q0 = a->tile_q0;
  p.G = a->num_q_heads / a->num_kv_heads; p.head_begin = 0;
  p.block_size = a->block_size > 0 ? a->block_size : 16; p.window_left = a->window_left;
  p.tiles_per_block = p.block_size / 16;
  p.tpb_magic = (uint32_t)(((1ull << 31) + p.tiles_per_block - 1) / p.tiles_per_block);
  p.scale_log2 = a->scale * sb::kLog2e;
  p.q_sr = a->q_stride_row; p.q_sh = a->q_stride_head; p.o_sr = a->out_stride_row; p.o_sh = a->out_stride_head;
  p.kv_sb = a->kv_stride_block * kv_esz; p.kv_sr = a->kv_stride_row * kv_esz; p.kv_sh = a->kv_stride_head * kv_esz;
  p.k_scale = a->k_scale; p.v_scale = a->v_scale;
  p.k_scale_tensor = a->k_scale_tensor; p.v_scale_tensor = a->v_scale_tensor; p.Hkv = a->num_kv_heads;
  p.bt_stride = a->block_table_stride;
  p.num_tiles = (int)a->num_tiles;
  p.meta_k = p.meta_v = nullptr;
  p.meta_len = 0;
  p.meta_sr = p.meta_sh = 0;
  p.opt.on = 0;
  p.opt.slopes = nullptr;
  p.opt.cap = p.opt.inv_cap2_log2e = 0.f;
  p.opt.mult = a->scale;  // (byte-code rows are dequantised on their way into LDS: the scores are those of elements)
  p.opt.inv_mult = 1.f / p.opt.mult;
  if (a->softcap < 0.f || a->softcap != a->softcap) return fail(SB_ERR_INVALID, "sb_swa_prefill: softcap must be >= 0");
  p.meta_bias_off = 0;
  if (a->softcap > 0.f || a->alibi_slopes) {
    if (a->meta_len > 0) {
      if (a->meta_bias_row0 < 0 || a->meta_bias_rows <= 0 || a->meta_bias_rows > 0x3fffffffLL ||
          a->meta_bias_row0 > a->meta_bias_rows)
        return fail(SB_ERR_INVALID, "sb_swa_prefill: soft cap / ALiBi with meta tokens need meta_bias_rows (the query rows "
                                    "of the reference's stacked second attention) and meta_bias_row0 inside it");
      p.meta_bias_off = (int)(a->meta_bias_row0 + a->meta_len - a->meta_bias_rows);
    }
    p.opt.on = 1;
    p.opt.slopes = a->alibi_slopes;
    if (a->softcap > 0.f) {
      p.opt.cap = a->softcap;
      p.opt.inv_cap2_log2e = 2.f * sb::kLog2e / a->softcap;
    }
  }
  if (a->meta_len < 0) return fail(SB_ERR_INVALID, "sb_swa_prefill: negative meta_len");
  if (a->meta_len > 0) {
    if (!a->meta_k || !a->meta_v) return fail(SB_ERR_INVALID, "sb_swa_prefill: meta_len without meta_k / meta_v");
    if (((reinterpret_cast<uintptr_t>(a->meta_k) | reinterpret_cast<uintptr_t>(a->meta_v)) & 15u) ||
        (a->meta_stride_row * 2) % 16 || (a->meta_stride_head * 2) % 16)
      return fail(SB_ERR_INVALID, "sb_swa_prefill: meta rows must be 16-byte aligned");
    p.meta_k = (const char *)a->meta_k; p.meta_v = (const char *)a->meta_v;
    p.meta_len = a->meta_len;
    p.meta_sr = a->meta_stride_row * 2; p.meta_sh = a->meta_stride_head * 2;
  }

  const dim3 grid((unsigned)((a->num_tiles + 7) / 8 * 8), (unsigned)a->num_kv_heads);
  for (int h0 = 0; h0 < p.G; h0 += SB_PREFILL_HEADS) {  // a GQA group is covered SB_PREFILL_HEADS heads at a time
    p.head_begin = h0;
    const int nh = p.G - h0 < SB_PREFILL_HEADS ? p.G - h0 : SB_PREFILL_HEADS;
    if (a->dtype == SB_BF16) launch_prefill<BF16>(a->kv_quant, nh, grid, (hipStream_t)a->stream, p);
    else launch_prefill<F16>(a->kv_quant, nh, grid, (hipStream_t)a->stream, p);
    const int rc = check_launch("swa_prefill_kernel");
    if (rc != SB_OK) return rc;
  }
  return SB_OK;
}
