// Window-bounded single-query attention over a paged bf16/fp16 cache, split-K, matrix cores: the
// "stream" form of the split kernel. Same lane layouts and arithmetic as swa_decode_mfma.hip (S^T = K Q^T,
// O^T = V^T P^T with v_mfma_f32_16x16x32, P kept in the lane that computed it, V transposed in registers,
// online softmax in log2 units), but the work of a wavefront is ONE stream of items instead of a call per
// (row, run of chunks):
//
//   item  = one 32-key chunk of one query row: 16 loads (8 K and 8 V pieces of 16 bytes per lane) into one of
//           two register sets, then 16 matrix instructions and the softmax of 32 keys x 16 heads.
//   stream = the chunks of this workgroup's run, in order, whatever rows they belong to. While item i is
//           computed the loads of item i + 1 are in flight and the block-table entries of item i + 2 are
//           being looked up (scalar loads). A row boundary inside the run changes nothing in that
//           pattern: the first chunk of the next row is requested while the last chunk of this row is
//           computed; after that computation the row's partial result is stored and the accumulators start
//           again at zero. No pipeline drain, no refill with nothing in flight.
//
// Every item issues exactly the same number of vector loads, whether it is an interior chunk (wave-uniform
// base plus constant lane offsets), an edge chunk (first / last chunk of a window, or the chunk holding the
// key that a fused append has not written yet: rows clamped into the visible range, masked by their true
// index) or the first chunk of a new row. That is what keeps the waits exact: the compiler counts loads per
// path, and where paths that issued different numbers of loads meet it waits for the worst case, which in a
// software pipeline means waiting for the loads just issued. For the same reason what a row boundary adds
// (the partial result's stores, the next row's Q^T operands) is issued AFTER the computation of the row's last
// item, where it sits between two items' loads and is covered by the wait for the first of them (the Q^T
// operands fetched with every item instead, four more loads out of the cache, cost 5 % of the kernel), and the
// loads issued behind the end of a stream all go to one cached line (the per-segment kernel re-reads its last
// chunk there, 3 % of its traffic at the 7B decode shape).
//
// Runs. Fixed split (kBalanced = false): grid = (rows, kv-head groups, splits), a workgroup's run is
// chunks [cb, ce) of its row. Balanced split: the chunks of all rows are laid end to end and cut into
// gridDim.x runs that differ by one chunk at most; a run that covers several rows writes one partial per
// row, numbered workgroup + row, and the runs that start and end a row note their numbers for the merge.
// Every wavefront derives its run from seq_lens by itself (lane i looks at row base + i, one wave-wide
// scan); the rows of a batch of 64 are then read back from those lanes, so walking into the next row costs
// no memory access.
//
// Built for the serving path: paged cache, one query row per sequence, no key_lo, no meta rows. Everything
// else stays on the per-segment kernels of swa_decode_mfma.hip.
#include <type_traits>

#include <hip/hip_ext.h>

#include "common.h"
#include "mfma_util.h"
#include "swa_decode_params.h"

namespace {

using namespace sb;

constexpr float kNegInf = kNegInfF;

struct Slot {
  uint4 k0[4], k1[4];  // K operands of tile 0 / tile 1, one per 32-dim step
  uint4 v[8];          // V rows of this lane's 8 keys, dims 8c..8c+7
};

// What the computation of an item needs to know about it (wave-uniform).
struct Rec {
  int r, lo, hi, cc;
  bool row_first;  // the segment starts with the row's first chunk
  bool valid, edge, seg_last, row_last;
  int64_t part;  // index of the first head's partial of the segment (heads follow at part_hs)
};

__device__ __forceinline__ int stream_wave_scan(int x, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  return x;
}
__device__ __forceinline__ int stream_wave_sum(int x) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) x += __shfl_xor(x, d);
  return x;
}

template <typename E, bool kBalanced>
__global__ __launch_bounds__(256, 1) void swa_decode_stream_kernel(const DecodeParams p,
                                                                   const int32_t *__restrict__ block_table,
                                                                   const int32_t *__restrict__ seq_lens,
                                                                   const int64_t *__restrict__ slot_mapping,
                                                                   const int G, const int Hkv) {
  const int tid = threadIdx.x;
  const int kvh = blockIdx.y * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(tid >> 6);
  if (kvh >= Hkv) return;  // whole wavefront; there is no barrier in this kernel
  const int lane = tid & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int w = blockIdx.x;

  // ---- rows: lane i holds row batch0 + i ---------------------------------------------------------------
  int batch0 = 0;
  int v_lo = 0, v_hi = 0, v_n = 0, v_own = 0;
  // loads the 64 rows from `base` on; `before` = chunks of the rows below; returns the same for the next batch
  auto load_batch = [&](int base, int before) {
    const int rr = min(base + lane, p.rows - 1);
    int hi = seq_lens[rr];
    if (base + lane >= p.rows) hi = 0;
    const int lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
    v_lo = lo;
    v_hi = hi;
    v_n = hi > lo ? ((hi - 1) >> 5) - (lo >> 5) + 1 : 0;
    batch0 = base;
    if constexpr (kBalanced) {
      const int incl = stream_wave_scan(v_n, lane);
      v_own = before + incl - v_n;
      return before + __builtin_amdgcn_readlane(incl, 63);
    } else {
      return 0;
    }
  };

  // ---- this workgroup's run -------------------------------------------------------------------------------
  int c1 = 0;          // balanced: end of the run on the common chunk axis
  int axis_next = 0;   // balanced: chunks of the rows below batch0 + 64
  int i0, cb, ce;      // first segment: lane of its row, chunks [cb, ce)
  if constexpr (kBalanced) {
    int total = 0;
    if (p.rows > 64) {  // more rows than lanes: the total needs a pass of its own
      for (int base = 0; base < p.rows; base += 64) {
        const int rr = min(base + lane, p.rows - 1);
        int hi = seq_lens[rr];
        if (base + lane >= p.rows) hi = 0;
        const int lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
        const int nn = hi > lo ? ((hi - 1) >> 5) - (lo >> 5) + 1 : 0;
        total += stream_wave_sum(nn);
      }
      total = __builtin_amdgcn_readfirstlane(total);
    }
    axis_next = load_batch(0, 0);
    if (p.rows <= 64) total = axis_next;
    // run w = chunks [w total / n, (w + 1) total / n) of the common axis: the runs differ by one chunk at most
    const int n_wg = gridDim.x;
    // (fewer chunks than runs: one chunk each for the first `total` runs, so that no run in the middle of a row
    // is empty: the merge reads a partial from every run between a row's first and last)
    const int c0 = total < n_wg ? w : (int)((int64_t)w * total / n_wg);
    c1 = total < n_wg ? min(w + 1, total) : (int)((int64_t)(w + 1) * total / n_wg);
    if (c0 >= c1) return;
    while (axis_next <= c0) axis_next = load_batch(batch0 + 64, axis_next);  // (c0 < total: ends inside the rows)
    const uint64_t cand = __builtin_amdgcn_ballot_w64(v_n > 0 && v_own + v_n > c0);
    i0 = __builtin_ctzll(cand);
    const int own = __builtin_amdgcn_readlane(v_own, i0);
    if (own >= c1) return;  // (cannot happen: the row that holds chunk c0 starts at or below it)
    const int fc = __builtin_amdgcn_readlane(v_lo, i0) >> 5, n = __builtin_amdgcn_readlane(v_n, i0);
    cb = fc + max(c0 - own, 0);
    ce = fc + min(c1 - own, n);
  } else {
    const int r = blockIdx.x;
    load_batch(r & ~63, 0);
    i0 = r & 63;
    const int fc = __builtin_amdgcn_readlane(v_lo, i0) >> 5, n = __builtin_amdgcn_readlane(v_n, i0);
    const int cps = (n + p.n_split - 1) / p.n_split;
    cb = fc + (int)blockIdx.z * cps;
    ce = min(cb + cps, fc + n);
  }
  const bool direct = !kBalanced && p.n_split == 1;
  const int part_hs = kBalanced ? 1 : p.n_split;
  auto part_of = [&](int r) -> int64_t {
    return kBalanced ? (int64_t)(w + r) * p.Hq : (int64_t)r * p.Hq * p.n_split + (int)blockIdx.z;
  };

  // ---- per-lane constants ---------------------------------------------------------------------------------
  const int64_t head_off = (int64_t)kvh * p.kv_sh;
  const uint32_t kv_sr32 = (uint32_t)p.kv_sr;
  const uint32_t koff = c * kv_sr32 + g * 16;  // K row c of a tile at 16-byte piece g
  uint32_t voff[4];                            // V rows 4g+j of a tile at piece c
#pragma unroll
  for (int j = 0; j < 4; ++j) voff[j] = (4 * g + j) * kv_sr32 + c * 16;
  // Q^T operand of lane (g, c): head c of the group (lanes c >= G repeat the last head: their columns of the
  // score tile are computed and never stored), 16-byte pieces 4s+g
  const uint32_t qoff = (uint32_t)((int64_t)(kvh * G + min(c, G - 1)) * p.q_sh * 2) + g * 16;
  const float my_slope = (p.opt.slopes && c < G) ? p.opt.slopes[kvh * G + c] : 0.f;
  const bool fused = p.new_k != nullptr;
  const int tpb = p.block_size >> 4;  // 16-key tiles per block

  f32x4_t acc[8];
  float m, l;
  auto reset = [&]() {
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    m = kNegInf;
    l = 0.f;
  };
  reset();

  // ---- the front of the stream: the next item to be requested ---------------------------------------------
  bool f_valid = true;
  int f_i = i0, f_r, f_lo, f_hi, f_cc, f_ce, f_end;  // f_end: one past the last chunk of the row's window
  bool f_row_first = false;
  int f_blk0 = 0, f_blk1 = 0, f_in0 = 0, f_in1 = 0;  // the item's two tiles: block-table entry, first row inside the block
  bool f_edge = false;
  // Looks the blocks of the front item's tiles up. Only the loads are issued here; the entries are first
  // touched by the next issue(), a computation later (an address worked out on the spot would make the
  // wavefront wait for each lookup before it goes on to compute).
  auto locate = [&]() {
    f_edge = (f_cc << 5) < f_lo || (f_cc << 5) + 32 > f_hi || (fused && f_cc == ((f_hi - 1) >> 5));
    int t0 = 2 * f_cc, t1 = t0 + 1;
    if (f_edge) {
      const int first_tile = f_lo >> 4, last_tile = (f_hi - 1) >> 4;
      t0 = min(max(t0, first_tile), last_tile);
      t1 = min(max(t1, first_tile), last_tile);
    }
    const int bi0 = tpb == 1 ? t0 : t0 / tpb, bi1 = tpb == 1 ? t1 : t1 / tpb;
    const int32_t *row = block_table + (int64_t)f_r * p.bt_stride;
    f_in0 = (t0 - bi0 * tpb) << 4;
    f_in1 = (t1 - bi1 * tpb) << 4;
    f_blk0 = row[bi0];
    f_blk1 = row[bi1];
  };
  auto enter = [&](int i, int first, int last) {
    f_i = i;
    f_r = batch0 + i;
    f_lo = __builtin_amdgcn_readlane(v_lo, i);
    f_hi = __builtin_amdgcn_readlane(v_hi, i);
    f_end = (f_lo >> 5) + __builtin_amdgcn_readlane(v_n, i);
    f_row_first = first == (f_lo >> 5);
    f_cc = first;
    f_ce = last;
    locate();
  };
  auto advance = [&]() {
    if (!f_valid) return;
    if (++f_cc < f_ce) {
      locate();
      return;
    }
    if constexpr (!kBalanced) {
      f_valid = false;
    } else {
      for (;;) {
        const uint64_t later = f_i >= 63 ? 0ull : (~0ull << (f_i + 1));
        const uint64_t cand = __builtin_amdgcn_ballot_w64(v_n > 0) & later;
        if (cand) {
          const int i = __builtin_ctzll(cand);
          const int own = __builtin_amdgcn_readlane(v_own, i);
          if (own >= c1) {
            f_valid = false;
            return;
          }
          const int fc = __builtin_amdgcn_readlane(v_lo, i) >> 5, n = __builtin_amdgcn_readlane(v_n, i);
          enter(i, fc, fc + min(c1 - own, n));
          return;
        }
        if (batch0 + 64 >= p.rows || axis_next >= c1) {
          f_valid = false;
          return;
        }
        axis_next = load_batch(batch0 + 64, axis_next);
        f_i = -1;
      }
    }
  };
  auto snapshot = [&]() {
    Rec x;
    x.r = f_r; x.lo = f_lo; x.hi = f_hi; x.cc = f_cc;
    x.row_first = f_row_first;
    x.valid = f_valid;
    x.edge = f_edge;
    x.seg_last = f_cc + 1 == f_ce;
    x.row_last = f_cc + 1 == f_end;
    x.part = part_of(f_r);
    return x;
  };

  // ---- the 16 loads of the front item ---------------------------------------------------------------------
  // All of them in one straight line of code, after the (load-free) branch that works out the addresses:
  // where an interior and an edge path each issued their own loads, the compiler's wait counts had to allow
  // for a path that runs neither.
  // (`opaque` keeps the loads behind the address branch; the pointers stay in the global address space, or the
  // loads would become flat ones, which count as LDS accesses too)
  typedef const __attribute__((address_space(1))) char *gptr_t;
  auto opaque = [](gptr_t &ptr) { asm("" : "+v"(ptr)); };
  auto stream16 = [](gptr_t ptr) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x4_t *>(ptr));
    return make_uint4(v.x, v.y, v.z, v.w);
  };
  auto issue = [&](Slot &s) {
    const char *newk = p.new_k + (int64_t)f_r * p.nk_st + (int64_t)kvh * p.nk_sh;
    const char *newv = p.new_v + (int64_t)f_r * p.nv_st + (int64_t)kvh * p.nv_sh;
    const int64_t b0 = (int64_t)f_blk0 * p.kv_sb + (int64_t)f_in0 * p.kv_sr + head_off;
    const int64_t b1 = (int64_t)f_blk1 * p.kv_sb + (int64_t)f_in1 * p.kv_sr + head_off;
    const char *k0p = p.k + b0, *k1p = p.k + b1, *v0p = p.v + b0, *v1p = p.v + b1;
    const char *gk0, *gk1, *gv0[4], *gv1[4];
    if (!f_valid) {  // behind the end of the stream: the same 16 loads, all lanes on one line that the cache holds
      gk0 = gk1 = p.q;
#pragma unroll
      for (int j = 0; j < 4; ++j) gv0[j] = gv1[j] = p.q;
    } else if (!f_edge) {  // every key visible and in the cache: wave-uniform bases plus constant lane offsets
      gk0 = k0p + koff;
      gk1 = k1p + koff;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        gv0[j] = v0p + voff[j];
        gv1[j] = v1p + voff[j];
      }
    } else {
      // tiles and rows clamped into the visible range; the newest row comes from the step's key / value
      // tensors when the append is fused (it is not in the cache yet). Rows outside [lo, hi) are never read.
      const int first_tile = f_lo >> 4, last_tile = (f_hi - 1) >> 4;
      const int t0c = min(max(2 * f_cc, first_tile), last_tile), t1c = min(max(2 * f_cc + 1, first_tile), last_tile);
      auto clamp_row = [&](int tc, int row) { return min(max((tc << 4) + row, f_lo), f_hi - 1) - (tc << 4); };
      const int newest = fused ? f_hi - 1 : -1;
      const int r0 = clamp_row(t0c, c), r1 = clamp_row(t1c, c);
      gk0 = ((t0c << 4) + r0 == newest) ? newk + g * 16 : k0p + r0 * kv_sr32 + g * 16;
      gk1 = ((t1c << 4) + r1 == newest) ? newk + g * 16 : k1p + r1 * kv_sr32 + g * 16;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int q0 = clamp_row(t0c, 4 * g + j), q1 = clamp_row(t1c, 4 * g + j);
        gv0[j] = ((t0c << 4) + q0 == newest) ? newv + c * 16 : v0p + q0 * kv_sr32 + c * 16;
        gv1[j] = ((t1c << 4) + q1 == newest) ? newv + c * 16 : v1p + q1 * kv_sr32 + c * 16;
      }
    }
    gptr_t pk0 = (gptr_t)gk0, pk1 = (gptr_t)gk1, pv0[4], pv1[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      pv0[j] = (gptr_t)gv0[j];
      pv1[j] = (gptr_t)gv1[j];
    }
    opaque(pk0);
    opaque(pk1);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      opaque(pv0[j]);
      opaque(pv1[j]);
    }
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      s.k0[st] = stream16(pk0 + st * 64);
      s.k1[st] = stream16(pk1 + st * 64);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s.v[j] = stream16(pv0[j]);
      s.v[4 + j] = stream16(pv1[j]);
    }
  };

  // ---- one item: S^T = K Q^T, online softmax, O^T += V^T P^T ---------------------------------------------
  // ---- what belongs to a row, not to an item: its Q^T operands and, for a fused append, 16 bytes of its new
  // K (lanes 0..15) / V (lanes 16..31) row. Loaded when the stream starts and, for the next row, at the end
  // of a segment BEHIND that segment's last computation and stores: there the four or five loads sit between
  // the loads of the next item and of the one after it, and the wait for the next item's operands covers them.
  uint4 qb[4], fresh;
  auto load_row = [&](int r) {
    const char *qrow = p.q + (int64_t)r * p.q_sr * 2;
#pragma unroll
    for (int st = 0; st < 4; ++st) qb[st] = *reinterpret_cast<const uint4 *>(qrow + qoff + st * 64);
    if (fused) {
      const char *newk = p.new_k + (int64_t)r * p.nk_st + (int64_t)kvh * p.nk_sh;
      const char *newv = p.new_v + (int64_t)r * p.nv_st + (int64_t)kvh * p.nv_sh;
      fresh = *reinterpret_cast<const uint4 *>((lane < 16 ? newk : newv) + (lane & 15) * 16);
    }
  };
  auto compute = [&](const Rec &x, const Slot &s) {
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      s0 = Mma<E>::run(s.k0[st], qb[st], s0);
      s1 = Mma<E>::run(s.k1[st], qb[st], s1);
    }
    float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
    const int i0k = x.cc << 5;
    if (p.opt.on) {  // soft cap / ALiBi (wave-uniform; the query sits at key index hi - 1)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        sc[j] = adjust_score(p.opt, sc[j], my_slope, (float)(i0k + ((j >> 2) << 4) + 4 * g + (j & 3) - (x.hi - 1)));
    }
    if (x.edge) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int i = i0k + ((j >> 2) << 4) + 4 * g + (j & 3);
        if (i < x.lo || i >= x.hi) sc[j] = kNegInf;
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
    for (int mt = 0; mt < 8; ++mt) acc[mt] = Mma<E>::run(v_transposed(s.v, mt), pb, acc[mt]);
  };

  // ---- end of a segment: the partial result (or the row's output), the fused append, a fresh start --------
  auto finish = [&](const Rec &x, bool any, const Rec &next) {
    if (fused && any && x.row_last && lane < 32) {  // store the newest K/V row at its slot (its bytes came with the row's Q)
      const int64_t slot = slot_mapping[x.r];  // (a scalar load: the pointer is restrict-qualified)
      if (slot >= 0) {
        const int64_t blk = slot / p.block_size;
        const int64_t dst = blk * p.kv_sb + (slot - blk * p.block_size) * p.kv_sr + head_off + (lane & 15) * 16;
        *reinterpret_cast<uint4 *>(const_cast<char *>(lane < 16 ? p.k : p.v) + dst) = fresh;
      }
    }
    if constexpr (kBalanced) {
      // the runs that start and end a row tell the merge which runs hold the row's partials: every run from
      // the first to the last (rows without chunks have none; the merge sees that from the row's length)
      if (any && kvh == 0 && lane == 0) {
        if (x.row_first) p.ws_rows[2 * x.r] = w;
        if (x.row_last) p.ws_rows[2 * x.r + 1] = w;
      }
    }
    float lt = l;
    lt += __shfl_xor(lt, 16);
    lt += __shfl_xor(lt, 32);
    if (c < G) {  // lane (g, c < G) owns head c, dims 32g + 8i + mt
      const int hq = kvh * G + c;
      if (direct) {
        const float inv = lt > 0.f ? 1.f / lt : 0.f;
        char *dst = p.out + ((int64_t)x.r * p.o_sr + (int64_t)hq * p.o_sh + 32 * g) * 2;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint4 o;
          o.x = E::pack(acc[0][i] * inv, acc[1][i] * inv);
          o.y = E::pack(acc[2][i] * inv, acc[3][i] * inv);
          o.z = E::pack(acc[4][i] * inv, acc[5][i] * inv);
          o.w = E::pack(acc[6][i] * inv, acc[7][i] * inv);
          *reinterpret_cast<uint4 *>(dst + 16 * i) = o;
        }
        if (g == 0 && p.lse) p.lse[(int64_t)x.r * p.Hq + hq] = lt > 0.f ? (m + log2f(lt)) * kLn2 : kNegInf;
      } else {
        const int64_t part = x.part + (int64_t)hq * part_hs;
        float *dst = p.ws_acc + part * 128 + 32 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          reinterpret_cast<float4 *>(dst + 8 * i)[0] = make_float4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]);
          reinterpret_cast<float4 *>(dst + 8 * i)[1] = make_float4(acc[4][i], acc[5][i], acc[6][i], acc[7][i]);
        }
        if (g == 0) {
          p.ws_ml[part * 2] = m;
          p.ws_ml[part * 2 + 1] = lt;
        }
      }
    }
    reset();
    if (any && next.valid) load_row(next.r);
  };

  if (cb >= ce) {  // fixed split: a part of the row with no chunks still owes the merge its (empty) partial
    Rec x;
    x.r = batch0 + i0; x.lo = x.hi = x.cc = 0;
    x.row_first = false;
    x.valid = true;
    x.edge = x.seg_last = x.row_last = false;
    x.part = part_of(x.r);
    finish(x, false, x);
    return;
  }

  // ---- the stream ---------------------------------------------------------------------------------------------
  // Two items per turn of the loop, one per register set, and no way out of the loop but its end: an exit
  // from the middle would add a path on which the second set's loads are still in flight when the first half
  // runs again, and the compiler would then wait for everything in flight before touching a register of
  // that set. A stream with an odd number of items ends with an empty item (valid = false: 16 loads of one
  // cached line, nothing computed).
  Slot ring[2];
  Rec rec0, rec1;
  enter(i0, cb, ce);
  rec0 = snapshot();
  load_row(rec0.r);
  issue(ring[0]);
  advance();
  do {
    rec1 = snapshot();
    issue(ring[1]);
    advance();
    compute(rec0, ring[0]);
    if (rec0.seg_last) finish(rec0, true, rec1);
    rec0 = snapshot();
    issue(ring[0]);
    advance();
    if (rec1.valid) {
      compute(rec1, ring[1]);
      if (rec1.seg_last) finish(rec1, true, rec0);
    }
  } while (rec0.valid);
}

}  // namespace

namespace sb_host {

// Launches the stream form of the matrix-core split kernel (bf16 / fp16, paged cache, one query row per
// sequence). p.n_wg > 0: balanced split with p.n_wg workgroups per kv-head group; else grid (rows, groups, splits).
// ev_start / ev_stop (both or neither): HIP events on the kernel's own dispatch.
void launch_swa_decode_stream(int dtype, int G, int Hkv, unsigned rows, unsigned n_split, hipStream_t st,
                              const sb::DecodeParams &p, hipEvent_t ev_start, hipEvent_t ev_stop) {
  const int waves = Hkv < 4 ? Hkv : 4;  // one wavefront (kv head) per SIMD, each with the whole register file
  const unsigned ygroups = (unsigned)((Hkv + waves - 1) / waves);
  const dim3 block(64 * waves);
  const bool timed = ev_start && ev_stop;
#define SB_STREAM(E, BAL, GRID)                                                                                        \
  do {                                                                                                                 \
    if (timed)                                                                                                         \
      hipExtLaunchKernelGGL((swa_decode_stream_kernel<E, BAL>), GRID, block, 0, st, ev_start, ev_stop, 0, p,           \
                            p.block_table, p.seq_lens, p.slot_mapping, G, Hkv);                                                        \
    else                                                                                                               \
      hipLaunchKernelGGL((swa_decode_stream_kernel<E, BAL>), GRID, block, 0, st, p, p.block_table, p.seq_lens, p.slot_mapping, G, Hkv); \
  } while (0)
  if (p.n_wg > 0) {
    const dim3 grid((unsigned)p.n_wg, ygroups);
    if (dtype == SB_BF16) SB_STREAM(sb::BF16, true, grid);
    else SB_STREAM(sb::F16, true, grid);
  } else {
    const dim3 grid(rows, ygroups, n_split);
    if (dtype == SB_BF16) SB_STREAM(sb::BF16, false, grid);
    else SB_STREAM(sb::F16, false, grid);
  }
#undef SB_STREAM
}

}  // namespace sb_host
