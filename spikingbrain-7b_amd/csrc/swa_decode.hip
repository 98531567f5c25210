// Window-bounded single-query attention over a paged (or dense) KV cache, split-K.
//
// Work decomposition
//   grid = (query rows, kv heads, splits); one 256-thread workgroup (4 wavefronts) handles
//   one kv head of one query row over one contiguous part of the visible window, for all G
//   query heads of the GQA group at once, so every K/V byte is fetched from HBM once and
//   used G times.
//   The window is cut into tiles of 16 keys (a vLLM cache block is a whole number of tiles).
//   Inside a wavefront lane = (g, c): c = lane%16 owns head dims [8c, 8c+8) (one 16-byte
//   vector of a bf16 row), g = lane/16 picks one of the 4 key rows a load instruction covers,
//   so one instruction fetches 4 whole 256-byte rows. Partial dot products are all-reduced
//   over the 16 lanes of a row with DPP; each of the 4 row groups keeps its own online-softmax
//   state (m, l, acc[G][8]) and the 16 row groups of a workgroup are merged once at the end
//   (registers -> LDS), then either normalised and stored (n_split == 1) or written as an
//   fp32 partial (m, l, acc) that swa_decode_merge_kernel combines.
//   Scores are kept in log2 units: p = exp2(s*scale*log2e - m).
//   Head sizes other than 128 (the reference's backend lists 32 .. 256 in steps of 32,
//   vllm_hymeta/attention/meta_attention.py:57-59) run this kernel with LPR = 8 or 32 lanes per row instead of
//   16 (a load instruction then covers 8 or 2 rows); lanes past the head's last dim carry zeros.
#include <algorithm>
#include <functional>
#include <mutex>
#include <queue>
#include <vector>

#include "common.h"
#include "swa_decode_params.h"

namespace sb_host {
void launch_swa_decode_split_mfma(int dtype, int G, int Hkv, unsigned rows, unsigned n_split, int depth,
                                  hipStream_t st, const sb::DecodeParams &p, hipEvent_t ev_start, hipEvent_t ev_stop);
void launch_swa_decode_stream(int dtype, int G, int Hkv, unsigned rows, unsigned n_split, hipStream_t st,
                              const sb::DecodeParams &p, hipEvent_t ev_start, hipEvent_t ev_stop);
void launch_swa_decode_split_i8(int dtype, int kv_quant, int G, int Hkv, unsigned rows, unsigned n_split, hipStream_t st,
                                const sb::DecodeParams &p);
}

namespace {

using namespace sb;

template <typename E>
struct Pack {
  uint32_t w[E::kPackWords];
};

template <typename E>
__device__ __forceinline__ Pack<E> load_pack(const char *p) {
  Pack<E> r;
  const uint4 a = *reinterpret_cast<const uint4 *>(p);
  r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w;
  if constexpr (E::kPackWords == 8) {
    const uint4 b = *reinterpret_cast<const uint4 *>(p + 16);
    r.w[4] = b.x; r.w[5] = b.y; r.w[6] = b.z; r.w[7] = b.w;
  }
  return r;
}

template <typename E>
__device__ __forceinline__ float dot_pack(const Pack<E> &a, const Pack<E> &b) {
  float s = 0.f;
  if constexpr (E::kPackWords == 8) {
#pragma unroll
    for (int i = 0; i < 8; ++i) s = fmaf(__uint_as_float(a.w[i]), __uint_as_float(b.w[i]), s);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) s = E::dot2(a.w[i], b.w[i], s);
  }
  return s;
}

template <typename E>
__device__ __forceinline__ void unpack(const Pack<E> &a, float (&f)[8]) {
  if constexpr (E::kPackWords == 8) {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = __uint_as_float(a.w[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = E::lo(a.w[i]);
      f[2 * i + 1] = E::hi(a.w[i]);
    }
  }
}

template <typename E>
__device__ __forceinline__ void store_out(char *out, int64_t idx, float x) {
  if constexpr (E::kPackWords == 8) {
    reinterpret_cast<float *>(out)[idx] = x;
  } else {
    reinterpret_cast<uint16_t *>(out)[idx] = (uint16_t)(E::pack(x, 0.f) & 0xffffu);
  }
}

constexpr float kNegInf = -__builtin_inff();

// sum over each aligned group of LPR lanes
template <int LPR>
__device__ __forceinline__ float row_allreduce_sum(float v) {
  if constexpr (LPR == 16) {
    return row16_allreduce_sum(v);
  } else {
#pragma unroll
    for (int o = 1; o < LPR; o <<= 1) v += __shfl_xor(v, o);
    return v;
  }
}

// LPR: lanes per key row (8 dims each; head sizes up to 8 LPR). NJ load instructions of 64 / LPR rows cover a tile.
template <typename E, int G, int LPR>
__global__ __launch_bounds__(256) void swa_decode_split_kernel(const DecodeParams p) {
  constexpr int kPackBytes = 8 * E::kBytes;
  constexpr bool kPrefetch = (E::kBytes == 2);
  constexpr int RPL = 64 / LPR, NJ = 16 / RPL;

  const int64_t r = blockIdx.x;
  // a GQA group of p.group_parts * G query heads is served by p.group_parts workgroups of G heads each
  const int kvh = blockIdx.y / p.group_parts;
  const int head0 = kvh * (p.group_parts * G) + (blockIdx.y - kvh * p.group_parts) * G;
  const int split = blockIdx.z;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int g = lane / LPR;
  const int c_lane = lane % LPR;
  // lanes past the head's last dim (head sizes that do not fill the LPR lanes) work on the last 8 dims with a zero
  // query: their scores add nothing and their outputs are not stored
  const bool live = c_lane * 8 < p.D;
  const int c = live ? c_lane : p.D / 8 - 1;

  const int64_t seq = p.row_seq ? (int64_t)p.row_seq[r] : r;
  const int hi = p.seq_lens[r];
  int lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
  if (p.key_lo) lo = max(lo, p.key_lo[r]);

  const int first_tile = lo >> 4;
  const int n_tiles = hi > lo ? ((hi - 1) >> 4) - first_tile + 1 : 0;
  const int tps = (n_tiles + p.n_split - 1) / p.n_split;
  const int tb = first_tile + split * tps;
  const int te = min(tb + tps, first_tile + n_tiles);

  // query vectors of the group, this lane's 8 dims
  Pack<E> qp[G];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    qp[h] = load_pack<E>(p.q + (r * p.q_sr + (int64_t)(head0 + h) * p.q_sh + c * 8) * E::kBytes);
    if (!live) {
#pragma unroll
      for (int i = 0; i < E::kPackWords; ++i) qp[h].w[i] = 0u;
    }
  }

  float slope[G];  // ALiBi slopes of the group's heads
#pragma unroll
  for (int h = 0; h < G; ++h) slope[h] = p.opt.slopes ? p.opt.slopes[head0 + h] : 0.f;

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m[h] = kNegInf;
    l[h] = 0.f;
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[h][d] = 0.f;
  }

  const bool paged = p.block_table != nullptr;
  const int64_t dense_row0 = (!paged && p.kv_start) ? p.kv_start[seq] : 0;
  const int64_t lane_off = (int64_t)kvh * p.kv_sh + c * kPackBytes;

  // byte offset of the first row of tile t (uniform over the wavefront); callers pass t < te
  auto tile_base = [&](int t) -> int64_t {
    const int i0 = t << 4;
    if (paged) {
      const int bi = i0 / p.block_size;
      const int64_t blk = p.block_table[seq * p.bt_stride + bi];
      return blk * p.kv_sb + (int64_t)(i0 - bi * p.block_size) * p.kv_sr;
    }
    return (dense_row0 + i0) * p.kv_sr;
  };
  // rows outside [lo, hi) are clamped onto the nearest visible key: nothing outside the window
  // is ever read, so stale or uninitialised rows cannot leak in through 0 * NaN
  auto load_tile = [&](int t, int64_t base, Pack<E> (&kb)[NJ], Pack<E> (&vb)[NJ]) {
    const int i0 = t << 4;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int row = min(max(RPL * j + g, lo - i0), hi - 1 - i0);
      const int64_t off = base + (int64_t)row * p.kv_sr + lane_off;
      kb[j] = load_pack<E>(p.k + off);
      vb[j] = load_pack<E>(p.v + off);
    }
  };

  // tile t of the window (keys [lo, hi) visible), or, with `meta`, of the meta rows (rows [0, meta_len) visible)
  auto compute_tile = [&](int t, const Pack<E> (&kb)[NJ], const Pack<E> (&vb)[NJ], const bool meta) {
    const int i0 = t << 4;
    const int vis_lo = meta ? 0 : lo, vis_hi = meta ? p.meta_len : hi;
    float s[G][NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int h = 0; h < G; ++h) s[h][j] = row_allreduce_sum<LPR>(dot_pack<E>(qp[h], kb[j]));
    if (p.opt.on) {  // soft cap / ALiBi (wave-uniform; the query sits at key index hi - 1; a meta row's distance
                     // is that of the reference's stacked second attention)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int key = i0 + RPL * j + g;
        const float dist = meta ? -fabsf((float)(p.meta_bias_off + (int)r - key)) : (float)(key - (hi - 1));
#pragma unroll
        for (int h = 0; h < G; ++h) s[h][j] = adjust_score(p.opt, s[h][j], slope[h], dist);
      }
    }
    if (i0 < vis_lo || i0 + 16 > vis_hi) {  // edge tile: mask keys outside the visible range
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int i = i0 + RPL * j + g;
        if (i < vis_lo || i >= vis_hi) {
#pragma unroll
          for (int h = 0; h < G; ++h) s[h][j] = kNegInf;
        }
      }
    }
    float alpha[G];
    bool grew = false;
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float mx;
      if constexpr (NJ == 4) {
        mx = fmaxf(fmaxf(s[h][0], s[h][1]), fmaxf(s[h][2], s[h][3]));
      } else {
        mx = s[h][0];
#pragma unroll
        for (int j = 1; j < NJ; ++j) mx = fmaxf(mx, s[h][j]);
      }
      mx *= p.scale_log2;
      const float m_new = fmaxf(m[h], mx);
      const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
      grew |= (m_new > m[h]);
      alpha[h] = fast_exp2(m[h] - m_safe);
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        s[h][j] = fast_exp2(fmaf(s[h][j], p.scale_log2, -m_safe));
        psum += s[h][j];
      }
      l[h] = fmaf(l[h], alpha[h], psum);
      m[h] = m_new;
    }
    if (__builtin_amdgcn_ballot_w64(grew) != 0) {
#pragma unroll
      for (int h = 0; h < G; ++h)
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[h][d] *= alpha[h];
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      float vf[8];
      unpack<E>(vb[j], vf);
#pragma unroll
      for (int h = 0; h < G; ++h)
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[h][d] = fmaf(s[h][j], vf[d], acc[h][d]);
    }
  };

  int t = tb + wave;
  if constexpr (kPrefetch) {
    // Software pipeline, one tile deep: the loads of the next tile are issued before the
    // current tile is computed. The prefetch is unconditional (past the end it re-reads the
    // last tile of the split) so that the number of loads in flight is the same on every
    // path and the wait before the compute only covers the current tile's loads.
    if (t < te) {
      const int last = te - 1;
      Pack<E> kb[NJ], vb[NJ];
      load_tile(t, tile_base(t), kb, vb);
      int64_t base1 = tile_base(min(t + 4, last));
      for (; t < te; t += 4) {
        const int64_t base2 = tile_base(min(t + 8, last));
        Pack<E> kn[NJ], vn[NJ];
        load_tile(min(t + 4, last), base1, kn, vn);
        compute_tile(t, kb, vb, false);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          kb[j] = kn[j];
          vb[j] = vn[j];
        }
        base1 = base2;
      }
    }
  } else {
    for (; t < te; t += 4) {
      Pack<E> kb[NJ], vb[NJ];
      load_tile(t, tile_base(t), kb, vb);
      compute_tile(t, kb, vb, false);
    }
  }
  // Meta tokens: 16-row tiles of the shared meta rows, dealt to the wavefronts of all splits in turn, go into the
  // same softmax (rows past the last one repeat it and are masked).
  if (p.meta_len > 0) {
    const int meta_tiles = (p.meta_len + 15) >> 4;
    const char *mk = p.meta_k + (int64_t)kvh * p.meta_sh + c * kPackBytes, *mv = p.meta_v + (int64_t)kvh * p.meta_sh + c * kPackBytes;
    for (int mt = split * 4 + wave; mt < meta_tiles; mt += 4 * p.n_split) {
      Pack<E> kb[NJ], vb[NJ];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int64_t off = (int64_t)min((mt << 4) + RPL * j + g, p.meta_len - 1) * p.meta_sr;
        kb[j] = load_pack<E>(mk + off);
        vb[j] = load_pack<E>(mv + off);
      }
      compute_tile(mt, kb, vb, true);
    }
  }

  // ---- merge the row groups of this wavefront ----------------------------------------
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const float mo = m[h];
    float M = mo;
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1) M = fmaxf(M, __shfl_xor(M, o));
    const float f = (mo == kNegInf) ? 0.f : fast_exp2(mo - M);
    float lv = l[h] * f;
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1) lv += __shfl_xor(lv, o);
    l[h] = lv;
    m[h] = M;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      float a = acc[h][d] * f;
#pragma unroll
      for (int o = LPR; o < 64; o <<= 1) a += __shfl_xor(a, o);
      acc[h][d] = a;
    }
  }

  // ---- merge the 4 wavefronts through LDS ---------------------------------------------
  __shared__ float s_m[4][G], s_l[4][G];
  __shared__ __attribute__((aligned(16))) float s_acc[4][G][8 * LPR];
  if (g == 0 && live) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
      if (c == 0) {
        s_m[wave][h] = m[h];
        s_l[wave][h] = l[h];
      }
      float4 *dst = reinterpret_cast<float4 *>(&s_acc[wave][h][c * 8]);
      dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
      dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
    }
  }
  __syncthreads();
  for (int idx = tid; idx < G * p.D; idx += 256) {
    const int h = p.D == 128 ? idx >> 7 : idx / p.D, d = idx - h * p.D;
    const float M = fmaxf(fmaxf(s_m[0][h], s_m[1][h]), fmaxf(s_m[2][h], s_m[3][h]));
    float tot = 0.f, L = 0.f;
    if (M != kNegInf) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float mw = s_m[w][h];
        const float f = (mw == kNegInf) ? 0.f : fast_exp2(mw - M);
        tot = fmaf(s_acc[w][h][d], f, tot);
        L = fmaf(s_l[w][h], f, L);
      }
    }
    const int hq = head0 + h;
    if (p.n_split == 1) {
      store_out<E>(p.out, r * p.o_sr + (int64_t)hq * p.o_sh + d, L > 0.f ? tot / L : 0.f);
      if (d == 0 && p.lse) p.lse[r * p.Hq + hq] = L > 0.f ? (M + log2f(L)) * kLn2 : kNegInf;
    } else {
      const int64_t part = (r * p.Hq + hq) * p.n_split + split;
      p.ws_acc[part * p.D + d] = tot;
      if (d == 0) {
        p.ws_ml[part * 2] = M;
        p.ws_ml[part * 2 + 1] = L;
      }
    }
  }
}

// One workgroup of head_size threads per (query row, query head): log-sum-exp merge of the splits.
template <typename E>
__global__ __launch_bounds__(256) void swa_decode_merge_kernel(const DecodeParams p) {
  const int64_t rh = blockIdx.x;  // r*Hq + hq
  const int64_t r = rh / p.Hq;
  const int hq = (int)(rh - r * p.Hq);
  const int d = threadIdx.x;
  const float *ml = p.ws_ml + rh * p.n_split * 2;
  const float *acc = p.ws_acc + rh * p.n_split * p.D + d;
  // Four splits per trip, every load of a trip issued before any is used: with the usual split counts
  // the kernel is one round trip to memory. Across trips the running sums are rescaled to the new maximum.
  float tot = 0.f, L = 0.f, M = kNegInf;
  for (int s0 = 0; s0 < p.n_split; s0 += 4) {
    float ms[4], ls[4], av[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = min(s0 + j, p.n_split - 1);
      ms[j] = ml[2 * s];
      ls[j] = ml[2 * s + 1];
      av[j] = acc[(int64_t)s * p.D];
    }
    float Mn = M;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (s0 + j < p.n_split) Mn = fmaxf(Mn, ms[j]);
    if (Mn != kNegInf) {
      const float keep = (M == kNegInf) ? 0.f : fast_exp2(M - Mn);
      tot *= keep;
      L *= keep;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float f = (s0 + j >= p.n_split || ms[j] == kNegInf) ? 0.f : fast_exp2(ms[j] - Mn);
        tot = fmaf(av[j], f, tot);
        L = fmaf(ls[j], f, L);
      }
    }
    M = Mn;
  }
  store_out<E>(p.out, r * p.o_sr + (int64_t)hq * p.o_sh + d, L > 0.f ? tot / L : 0.f);
  if (d == 0 && p.lse) p.lse[rh] = L > 0.f ? (M + log2f(L)) * kLn2 : kNegInf;
}

// Merge for the balanced split: the partials of row r are numbers w + r for the workgroups w whose
// runs of chunks touch the row; which those are follows from seq_lens exactly as in the split kernel.
template <typename E>
__global__ __launch_bounds__(128) void swa_decode_merge_balanced_kernel(const DecodeParams p) {
  const int64_t rh = blockIdx.x;  // r*Hq + hq
  const int r = (int)(rh / p.Hq);
  const int hq = (int)(rh - (int64_t)r * p.Hq);
  const int d = threadIdx.x;
  const int lane = d & 63;
  int total = 0, before = 0;
  for (int base = 0; base < p.rows; base += 64) {
    const int rr = base + lane;
    int n = 0;
    if (rr < p.rows) {
      const int hi = p.seq_lens[rr];
      int lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
      if (p.key_lo) lo = max(lo, p.key_lo[rr]);
      n = hi > lo ? ((hi - 1) >> 5) - (lo >> 5) + 1 : 0;
    }
    const int len = n > 0 ? n + kBalancedRowStartChunks : 0;  // as the split kernel lays the rows out
    int t = len, b = rr < r ? len : 0;
#pragma unroll
    for (int k = 1; k < 64; k <<= 1) {
      t += __shfl_xor(t, k);
      b += __shfl_xor(b, k);
    }
    total += t;
    before += b;
  }
  int n_r = 0;
  {
    const int hi = p.seq_lens[r];
    int lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
    if (p.key_lo) lo = max(lo, p.key_lo[r]);
    n_r = hi > lo ? ((hi - 1) >> 5) - (lo >> 5) + 1 : 0;
  }
  float tot = 0.f, L = 0.f, M = kNegInf;
  if (n_r > 0) {
    const int per = (total + p.n_wg - 1) / p.n_wg;
    const int own = before + kBalancedRowStartChunks;          // the row's own chunks start behind its virtual ones
    const int w_lo = own / per, w_hi = (own + n_r - 1) / per;
    // a long row among short ones can have hundreds of partials: loads go out eight at a time
    for (int w = w_lo; w <= w_hi; w += 8) {
      float ms[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) ms[j] = p.ws_ml[((int64_t)(min(w + j, w_hi) + r) * p.Hq + hq) * 2];
#pragma unroll
      for (int j = 0; j < 8; ++j) M = fmaxf(M, ms[j]);
    }
    if (M != kNegInf) {
      for (int w = w_lo; w <= w_hi; w += 8) {
        float ms[8], ls[8], av[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int64_t part = (int64_t)(min(w + j, w_hi) + r) * p.Hq + hq;
          ms[j] = p.ws_ml[part * 2];
          ls[j] = p.ws_ml[part * 2 + 1];
          av[j] = p.ws_acc[part * 128 + d];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float f = (w + j > w_hi || ms[j] == kNegInf) ? 0.f : fast_exp2(ms[j] - M);
          tot = fmaf(av[j], f, tot);
          L = fmaf(ls[j], f, L);
        }
      }
    }
  }
  store_out<E>(p.out, (int64_t)r * p.o_sr + (int64_t)hq * p.o_sh + d, L > 0.f ? tot / L : 0.f);
  if (d == 0 && p.lse) p.lse[rh] = L > 0.f ? (M + log2f(L)) * kLn2 : kNegInf;
}

// Merge behind the stream form of the balanced split: the wavefront that ended a row has left the span of runs
// (workgroups) holding the row's partials in ws_rows, so nothing has to be worked out from the other rows'
// lengths here. Same arithmetic and order as swa_decode_merge_balanced_kernel.
template <typename E>
__global__ __launch_bounds__(128) void swa_decode_merge_rows_kernel(const DecodeParams p) {
  const int64_t rh = blockIdx.x;  // r*Hq + hq
  const int r = (int)(rh / p.Hq);
  const int hq = (int)(rh - (int64_t)r * p.Hq);
  const int d = threadIdx.x;
  const int hi = p.seq_lens[r];
  const int lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
  float tot = 0.f, L = 0.f, M = kNegInf;
  if (hi > lo) {
    const int w_lo = p.ws_rows[2 * r], w_hi = p.ws_rows[2 * r + 1];
    // eight partials per trip to memory, maxima, denominators and numerators together (a row cut into more
    // than eight runs goes round again and rescales what it has): one trip for almost every row
    for (int w = w_lo; w <= w_hi; w += 8) {
      float ms[8], ls[8], av[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int64_t part = (int64_t)(min(w + j, w_hi) + r) * p.Hq + hq;
        ms[j] = p.ws_ml[part * 2];
        ls[j] = p.ws_ml[part * 2 + 1];
        av[j] = p.ws_acc[part * 128 + d];
      }
      float Mn = M;
#pragma unroll
      for (int j = 0; j < 8; ++j) Mn = fmaxf(Mn, ms[j]);
      if (Mn != kNegInf) {
        const float keep = (M == kNegInf) ? 0.f : fast_exp2(M - Mn);
        tot *= keep;
        L *= keep;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float f = (w + j > w_hi || ms[j] == kNegInf) ? 0.f : fast_exp2(ms[j] - Mn);
          tot = fmaf(av[j], f, tot);
          L = fmaf(ls[j], f, L);
        }
      }
      M = Mn;
    }
  }
  store_out<E>(p.out, (int64_t)r * p.o_sr + (int64_t)hq * p.o_sh + d, L > 0.f ? tot / L : 0.f);
  if (d == 0 && p.lse) p.lse[rh] = L > 0.f ? (M + log2f(L)) * kLn2 : kNegInf;
}

struct LseMergeParams {
  char *out;
  float *lse;
  const char *block_out;
  const float *block_lse;
  int64_t pairs;  // rows * heads
  int heads, vecs;  // 8-element vectors per (row, head)
  int64_t o_sr, o_sh, b_sr, b_sh;  // elements
};

// One thread per 8 elements of a (row, head) pair. In log2-free form: with w = sigmoid(block_lse - lse),
// out' = out - w (out - block_out) and lse' = lse - logsigmoid(lse - block_lse) = max + log(1 + exp(-|d|)).
template <typename E>
__global__ __launch_bounds__(256) void lse_merge_kernel(const LseMergeParams p) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t pair = t / p.vecs;
  if (pair >= p.pairs) return;
  const int vec = (int)(t - pair * p.vecs);
  const int64_t r = pair / p.heads;
  const int h = (int)(pair - r * p.heads);
  const float la = p.lse[pair], lb = p.block_lse[pair];
  if (lb == kNegInf) return;  // nothing to merge in (also covers both sides empty)
  const float w = (la == kNegInf) ? 1.f : 1.f / (1.f + __expf(la - lb));
  constexpr int kEsz = E::kPackWords == 8 ? 4 : 2;
  char *op = p.out + (r * p.o_sr + (int64_t)h * p.o_sh + vec * 8) * kEsz;
  const char *bp = p.block_out + (r * p.b_sr + (int64_t)h * p.b_sh + vec * 8) * kEsz;
  float a[8], b[8];
  unpack<E>(load_pack<E>(op), a);
  unpack<E>(load_pack<E>(bp), b);
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = a[i] - w * (a[i] - b[i]);
  if constexpr (E::kPackWords == 8) {
    reinterpret_cast<float4 *>(op)[0] = make_float4(a[0], a[1], a[2], a[3]);
    reinterpret_cast<float4 *>(op)[1] = make_float4(a[4], a[5], a[6], a[7]);
  } else {
    *reinterpret_cast<uint4 *>(op) =
        make_uint4(E::pack(a[0], a[1]), E::pack(a[2], a[3]), E::pack(a[4], a[5]), E::pack(a[6], a[7]));
  }
  if (vec == 0) {
    const float hi = fmaxf(la, lb), lo = fminf(la, lb);
    p.lse[pair] = (lo == kNegInf) ? hi : hi + log1pf(__expf(lo - hi));
  }
}

template <typename E, int LPR>
int launch_for_group_lanes(int G, dim3 grid, hipStream_t st, const DecodeParams &p) {
  switch (G) {
    case 1: hipLaunchKernelGGL((swa_decode_split_kernel<E, 1, LPR>), grid, dim3(256), 0, st, p); return 0;
    case 2: hipLaunchKernelGGL((swa_decode_split_kernel<E, 2, LPR>), grid, dim3(256), 0, st, p); return 0;
    case 4: hipLaunchKernelGGL((swa_decode_split_kernel<E, 4, LPR>), grid, dim3(256), 0, st, p); return 0;
    case 7: hipLaunchKernelGGL((swa_decode_split_kernel<E, 7, LPR>), grid, dim3(256), 0, st, p); return 0;
    case 8: hipLaunchKernelGGL((swa_decode_split_kernel<E, 8, LPR>), grid, dim3(256), 0, st, p); return 0;
    default: return -1;
  }
}
// lanes per key row by head size: 8 (up to 64 dims), 16 (up to 128), 32 (up to 256)
template <typename E>
int launch_for_group(int G, dim3 grid, hipStream_t st, const DecodeParams &p) {
  if (p.D <= 64) return launch_for_group_lanes<E, 8>(G, grid, st, p);
  if (p.D <= 128) return launch_for_group_lanes<E, 16>(G, grid, st, p);
  return launch_for_group_lanes<E, 32>(G, grid, st, p);
}

inline int64_t round_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

}  // namespace

// Number of compute units of the current device (256 on MI355X); 256 if the query fails.
static int device_cu_count() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return 256;
  return cus;
}

// Cost model of a split launch, in units of one 32-key chunk streamed by one workgroup while every CU is
// busy (about 2.5 us), fitted to launches of 16 .. 384 window-saturated rows of the 7B shape:
//   fixed split    : rounds of workgroups over the CUs (one workgroup fits a CU at a time), each round
//                    costing its workgroups' chunks + kFixedChunks (start-up chain, partial result, launch
//                    and merge share); a last round that fills only part of the CUs runs up to 40 % faster;
//   balanced split : one run per CU + kBalancedChunks + rows / kBalancedRowsPerChunk (every wavefront adds
//                    up all rows' lengths, and the merge reads one more partial per row).
constexpr double kFixedChunks = 7.0;
constexpr double kBalancedChunks = 8.0;
constexpr double kBalancedRowsPerChunk = 25.0;

static double round_cost(double chunks_per_wg, int64_t active, int64_t cus) {
  const double fill = active >= cus ? 1.0 : (double)active / (double)cus;
  return (chunks_per_wg + kFixedChunks) * (0.6 + 0.4 * fill);
}

// Estimated duration of a fixed split of `wgs` (row, kv-head group) pairs of `chunks` chunks each into n
// parts on `cus` CUs.
static double split_cost(int64_t wgs, int64_t n, int64_t chunks, int64_t cus) {
  const int64_t total = wgs * n, full = total / cus, rest = total % cus;
  const double per_wg = (double)((chunks + n - 1) / n);
  return (double)full * round_cost(per_wg, cus, cus) + (rest ? round_cost(per_wg, rest, cus) : 0.0);
}

extern "C" int32_t sb_swa_decode_auto_split(int64_t num_rows, int32_t num_kv_heads,
                                            int32_t max_seq_len, int32_t window_left) {
  if (num_rows <= 0 || num_kv_heads <= 0 || max_seq_len <= 0) return 1;
  int64_t keys = max_seq_len;
  if (window_left >= 0 && keys > (int64_t)window_left + 1) keys = (int64_t)window_left + 1;
  const int64_t chunks = (keys + 31) / 32 + 1;  // +1: an unaligned window touches one more chunk
  // A split is one workgroup per (row, group of up to 4 kv heads). Take the split count with the lowest
  // estimated duration (rows x splits just above a multiple of the CU count pay a whole extra round),
  // leaving every workgroup at least 8 chunks (256 keys) so that its fixed cost stays small next to the
  // streaming; ties go to more splits (more CUs streaming).
  const int64_t wgs = num_rows * ((num_kv_heads + 3) / 4);
  const int64_t cus = device_cu_count();
  int64_t cap = chunks / 8;
  if (cap > 64) cap = 64;
  if (cap < 1) cap = 1;
  int64_t best = 1;
  double best_cost = split_cost(wgs, 1, chunks, cus);
  for (int64_t n = 2; n <= cap; ++n) {
    const double c = split_cost(wgs, n, chunks, cus);
    if (c <= best_cost) { best = n; best_cost = c; }
  }
  return (int32_t)best;
}

// Rows up to which the balanced split is used (every wavefront sums over all rows' lengths).
constexpr int64_t kBalancedMaxRows = 1024;

// Workgroups per kv-head group of the balanced split: one per CU (a CU holds one at a time), fewer only
// when the fixed split would have launched less than half as many (very little work).
static int64_t balanced_workgroups(int64_t num_rows, int64_t n_split) {
  const int64_t fixed = num_rows * n_split, cus = device_cu_count();
  return fixed * 2 >= cus ? cus : fixed;
}

// Partials of a launch: rows * n_split for the fixed split; the balanced split numbers them
// workgroup + row. Sized for whichever is larger.
static int64_t partial_slots(int64_t num_rows, int64_t n_split) {
  const int64_t fixed = num_rows * n_split;
  if (num_rows > kBalancedMaxRows) return fixed;
  const int64_t balanced = balanced_workgroups(num_rows, n_split) + num_rows;
  return balanced > fixed ? balanced : fixed;
}

extern "C" int32_t sb_swa_decode_prefer_balanced(const int32_t *host_seq_lens, int64_t num_rows,
                                                 int32_t window_left, int32_t n_split) {
  if (!host_seq_lens || num_rows <= 0 || num_rows > kBalancedMaxRows || n_split < 1) return 0;
  const int64_t cus = device_cu_count();
  std::vector<int64_t> chunks((size_t)num_rows);
  int64_t total = 0;
  for (int64_t r = 0; r < num_rows; ++r) {
    const int64_t hi = host_seq_lens[r];
    const int64_t lo = (window_left >= 0 && hi - 1 - window_left > 0) ? hi - 1 - window_left : 0;
    chunks[r] = hi > lo ? ((hi - 1) >> 5) - (lo >> 5) + 1 : 0;
    total += chunks[r];
  }
  // Fixed split: its workgroups (split-major, rows fastest: the dispatch order) handed to the CUs as
  // these fall free, one workgroup per CU at a time; each costs its chunks plus the fixed part.
  std::priority_queue<double, std::vector<double>, std::greater<double>> free_at;
  for (int64_t c = 0; c < cus; ++c) free_at.push(0.0);
  double fixed_end = 0.0;
  for (int64_t s = 0; s < n_split; ++s)
    for (int64_t r = 0; r < num_rows; ++r) {
      const int64_t cps = (chunks[r] + n_split - 1) / n_split;
      const int64_t mine = std::max<int64_t>(0, std::min(cps, chunks[r] - s * cps));
      const double end = free_at.top() + (double)mine + kFixedChunks;
      free_at.pop();
      free_at.push(end);
      if (end > fixed_end) fixed_end = end;
    }
  const int64_t n_wg = balanced_workgroups(num_rows, n_split < 2 ? 2 : n_split);
  int64_t nonempty = 0;
  for (int64_t r = 0; r < num_rows; ++r) nonempty += chunks[r] > 0;
  (void)nonempty;  // (the stream kernel, which serves these calls, charges a row start nothing)
  const double balanced_end = (double)((total + n_wg - 1) / n_wg) + kBalancedChunks + (double)num_rows / kBalancedRowsPerChunk;
  return balanced_end < fixed_end ? 1 : 0;
}

extern "C" size_t sb_swa_decode_workspace_bytes(int64_t num_rows, int32_t num_q_heads,
                                                int32_t head_size, int32_t n_split) {
  if (n_split <= 1 || num_rows <= 0 || num_q_heads <= 0 || head_size <= 0) return 0;
  const int64_t parts = partial_slots(num_rows, n_split) * num_q_heads;
  return (size_t)(kMergeCounterBytes + round_up(parts * head_size * 4, 256) + round_up(parts * 2 * 4, 256) +
                  round_up(num_rows * 2 * 4, 256));  // ... + per row the span of runs holding its partials (balanced split)
}

extern "C" int sb_swa_decode(const sb_swa_decode_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_swa_decode: null args");
  if (a->num_rows < 0) return fail(SB_ERR_INVALID, "sb_swa_decode: negative num_rows");
  if (a->num_rows == 0) return SB_OK;
  if (!a->q || !a->k_cache || !a->v_cache || !a->out || !a->seq_lens)
    return fail(SB_ERR_INVALID, "sb_swa_decode: null tensor pointer");
  // (vllm_hymeta/attention/meta_attention.py:57-59 lists 32 .. 256 in steps of 32; the matrix-core and byte-code
  // kernels are built for 128, the other sizes run on the vector kernel)
  if (a->head_size < 32 || a->head_size > 256 || a->head_size % 32 != 0)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: head_size %d (built: 32 to 256 in steps of 32)", a->head_size);
  if (a->head_size != 128 && a->kv_quant != SB_KV_NONE)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: byte-code caches are built for head_size 128 only");
  if (a->num_q_heads <= 0 || a->num_kv_heads <= 0 || a->num_q_heads % a->num_kv_heads != 0)
    return fail(SB_ERR_INVALID, "sb_swa_decode: num_q_heads must be a positive multiple of num_kv_heads");
  if (!(a->scale > 0.f)) return fail(SB_ERR_INVALID, "sb_swa_decode: scale must be positive");
  if (a->block_table && (a->block_size < 16 || a->block_size % 16 != 0))
    return fail(SB_ERR_INVALID, "sb_swa_decode: block_size %d must be a multiple of 16", a->block_size);
  if (a->num_rows > 0x7fffffffLL || a->num_kv_heads > 65535)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: grid too large");
  int esz;
  switch (a->dtype) {
    case SB_BF16:
    case SB_F16: esz = 2; break;
    case SB_F32: esz = 4; break;
    default: return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: unknown dtype %d", a->dtype);
  }
  const bool fp8_kv = a->kv_quant == SB_KV_FP8;
  const bool int8_kv = a->kv_quant == SB_KV_INT8 || fp8_kv;   // byte codes: the same kernel family
  if (a->kv_quant != SB_KV_NONE && !int8_kv)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: unknown kv_quant %d", a->kv_quant);
  if (fp8_kv && (!(a->k_scale_tensor > 0.f) || !(a->v_scale_tensor > 0.f)))
    return fail(SB_ERR_INVALID, "sb_swa_decode: the fp8 cache needs positive k_scale_tensor and v_scale_tensor");
  const int kv_esz = int8_kv ? 1 : esz;
  if (int8_kv) {
    if (a->dtype == SB_F32 || (a->flags & SB_DECODE_FORCE_VALU))
      return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: the INT8 cache needs bf16 or fp16 queries on the matrix-core path");
    if (!a->block_table || (!fp8_kv && (!a->k_scale || !a->v_scale)))
      return fail(SB_ERR_INVALID, "sb_swa_decode: the INT8 cache needs paged mode and both scale tensors");
    if (a->new_key || a->new_value || a->new_slot_mapping)
      return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: no fused append into the INT8 cache (call sb_kv_append_int8 first)");
    if (!fp8_kv && ((reinterpret_cast<uintptr_t>(a->k_scale) | reinterpret_cast<uintptr_t>(a->v_scale)) & 15u))
      return fail(SB_ERR_INVALID, "sb_swa_decode: scale tensors not 16-byte aligned");
  }
  const int64_t es[] = {a->q_stride_row, a->q_stride_head};
  for (int64_t s : es)
    if ((s * esz) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_swa_decode: stride %lld elements is not 16-byte aligned",
                  (long long)s);
  const int64_t kes[] = {a->kv_stride_block, a->kv_stride_row, a->kv_stride_head};
  for (int64_t s : kes)
    if ((s * kv_esz) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_swa_decode: cache stride %lld elements is not 16-byte aligned",
                  (long long)s);
  if ((reinterpret_cast<uintptr_t>(a->q) | reinterpret_cast<uintptr_t>(a->k_cache) |
       reinterpret_cast<uintptr_t>(a->v_cache)) & 15u)
    return fail(SB_ERR_INVALID, "sb_swa_decode: q/k/v base not 16-byte aligned");

  int n_split = a->n_split;
  if (n_split < 0) return fail(SB_ERR_INVALID, "sb_swa_decode: negative n_split");
  if (n_split == 0)
    n_split = sb_swa_decode_auto_split(a->num_rows, a->num_kv_heads, a->max_seq_len, a->window_left);
  if (n_split > 65535) return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: n_split > 65535");
  const size_t need = sb_swa_decode_workspace_bytes(a->num_rows, a->num_q_heads, a->head_size, n_split);
  if (need > 0 && (!a->workspace || a->workspace_bytes < need))
    return fail(SB_ERR_WORKSPACE, "sb_swa_decode: workspace of %zu bytes needed for n_split=%d, got %zu",
                need, n_split, a->workspace ? a->workspace_bytes : (size_t)0);
  if (need > 0 && (reinterpret_cast<uintptr_t>(a->workspace) & 15u))
    return fail(SB_ERR_INVALID, "sb_swa_decode: workspace not 16-byte aligned");

  DecodeParams p;
  p.q = (const char *)a->q; p.k = (const char *)a->k_cache; p.v = (const char *)a->v_cache;
  p.out = (char *)a->out; p.lse = a->lse;
  p.block_table = a->block_table; p.kv_start = a->kv_start; p.row_seq = a->row_seq;
  p.seq_lens = a->seq_lens; p.key_lo = a->key_lo;
  p.D = a->head_size;
  const int64_t parts = partial_slots(a->num_rows, n_split) * a->num_q_heads;
  // workspace = [arrival counters of the in-kernel merge | partial numerators | partial (max, denominator)]
  p.merge_counter = nullptr;
  p.Hkv = a->num_kv_heads;
  p.ws_acc = need ? (float *)((char *)a->workspace + kMergeCounterBytes) : nullptr;
  p.ws_ml = need ? (float *)((char *)a->workspace + kMergeCounterBytes + round_up(parts * a->head_size * 4, 256)) : nullptr;
  p.ws_rows = need ? (int32_t *)((char *)a->workspace + kMergeCounterBytes + round_up(parts * a->head_size * 4, 256) +
                                 round_up(parts * 2 * 4, 256)) : nullptr;
  p.Hq = a->num_q_heads; p.block_size = a->block_size > 0 ? a->block_size : 16;
  p.window_left = a->window_left; p.n_split = n_split;
  p.rows = (int)a->num_rows; p.n_wg = 0;
  p.scale_log2 = a->scale * sb::kLog2e;
  p.q_sr = a->q_stride_row; p.q_sh = a->q_stride_head;
  p.o_sr = a->out_stride_row; p.o_sh = a->out_stride_head;
  p.kv_sb = a->kv_stride_block * kv_esz; p.kv_sr = a->kv_stride_row * kv_esz; p.kv_sh = a->kv_stride_head * kv_esz;
  p.bt_stride = a->block_table_stride;
  p.k_scale = a->k_scale; p.v_scale = a->v_scale;
  p.kv_out_scale = 1.f;
  if (fp8_kv) {  // scores scale with the K tensor scale, the result with the V tensor scale
    p.scale_log2 *= a->k_scale_tensor;
    p.kv_out_scale = a->v_scale_tensor;
  }

  const int G = a->num_q_heads / a->num_kv_heads;
  const dim3 grid((unsigned)a->num_rows, (unsigned)a->num_kv_heads, (unsigned)n_split);
  hipStream_t st = (hipStream_t)a->stream;
  int rc = 0;
  if (a->phases < 0 || a->phases > 2) return fail(SB_ERR_INVALID, "sb_swa_decode: phases must be 0, 1 or 2");
  // bf16/fp16 at head size 128 run on the matrix cores (up to 16 query heads per kv head); everything else on the vector ALUs
  const bool mfma = (a->dtype != SB_F32) && !(a->flags & SB_DECODE_FORCE_VALU) && a->head_size == 128 && G <= 16;
  if (int8_kv && G > 16)
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: GQA group size %d over a byte-code cache (the matrix-core kernels take up to 16 query heads per kv head)", G);
  if (a->num_q_heads > 65535) return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: grid too large");
  // The vector kernel is built for 1, 2, 4, 7 and 8 query heads per workgroup; any other group size is cut
  // into parts of the largest of these that divides it (the parts read the same K/V rows).
  int vec_g = 1;
  for (int cand : {8, 7, 4, 2})
    if (G % cand == 0) { vec_g = cand; break; }
  p.group_parts = mfma ? 1 : G / vec_g;
  if (mfma && (a->kv_stride_row <= 0 || a->kv_stride_row * kv_esz * 16 >= (1LL << 31)))
    return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode: kv row stride %lld does not fit the kernel's 32-bit in-tile offsets",
                (long long)a->kv_stride_row);
  if (mfma && ((reinterpret_cast<uintptr_t>(a->out) & 15u) || (a->out_stride_row * esz) % 16 ||
               (a->out_stride_head * esz) % 16))
    return fail(SB_ERR_INVALID, "sb_swa_decode: out rows must be 16-byte aligned");

  // optional meta tokens: shared rows every query also attends to, inside the same softmax
  p.meta_k = p.meta_v = nullptr;
  p.meta_len = 0;
  p.meta_sr = p.meta_sh = 0;
  p.meta_k_mult = p.meta_v_mult = 1.f;
  if (a->meta_len < 0) return fail(SB_ERR_INVALID, "sb_swa_decode: negative meta_len");
  if (a->meta_len > 0) {
    if (!a->meta_k || !a->meta_v) return fail(SB_ERR_INVALID, "sb_swa_decode: meta_len without meta_k / meta_v");
    if ((mfma && (a->flags & SB_DECODE_BALANCED)) || (!mfma && int8_kv))
      return fail(SB_ERR_UNSUPPORTED,
                  "sb_swa_decode: meta tokens go with the fixed split (and, over a byte-code cache, with bf16/fp16 queries)");
    if (((reinterpret_cast<uintptr_t>(a->meta_k) | reinterpret_cast<uintptr_t>(a->meta_v)) & 15u) ||
        (a->meta_stride_row * esz) % 16 || (a->meta_stride_head * esz) % 16 || a->meta_stride_row <= 0)
      return fail(SB_ERR_INVALID, "sb_swa_decode: meta rows must be 16-byte aligned");
    p.meta_k = (const char *)a->meta_k; p.meta_v = (const char *)a->meta_v;
    p.meta_len = a->meta_len;
    p.meta_sr = a->meta_stride_row * esz; p.meta_sh = a->meta_stride_head * esz;
    if (fp8_kv) {
      p.meta_k_mult = 1.f / a->k_scale_tensor;
      p.meta_v_mult = 1.f / a->v_scale_tensor;
    }
  }
  // optional soft cap / ALiBi slopes on the scores
  p.opt.on = 0;
  p.opt.slopes = nullptr;
  p.opt.cap = p.opt.inv_cap2_log2e = 0.f;
  p.opt.mult = p.scale_log2 / sb::kLog2e;  // what turns a raw dot product into the scaled score (K tensor scale included)
  p.opt.inv_mult = 1.f / p.opt.mult;
  if (a->softcap < 0.f || a->softcap != a->softcap) return fail(SB_ERR_INVALID, "sb_swa_decode: softcap must be >= 0");
  p.meta_bias_off = 0;
  if (a->softcap > 0.f || a->alibi_slopes) {
    if (a->meta_len > 0) {
      const int64_t rows = a->meta_bias_rows > 0 ? a->meta_bias_rows : a->num_rows;
      const int64_t off = a->meta_bias_row0 + a->meta_len - rows;
      if (a->meta_bias_row0 < 0 || a->meta_bias_row0 + a->num_rows > rows || off > 0x3fffffffLL || off < -0x3fffffffLL)
        return fail(SB_ERR_INVALID, "sb_swa_decode: meta_bias_row0 %lld / meta_bias_rows %lld do not hold this call's %lld rows",
                    (long long)a->meta_bias_row0, (long long)a->meta_bias_rows, (long long)a->num_rows);
      p.meta_bias_off = (int)off;
    }
    p.opt.on = 1;
    p.opt.slopes = a->alibi_slopes;
    if (a->softcap > 0.f) {
      p.opt.cap = a->softcap;
      p.opt.inv_cap2_log2e = 2.f * sb::kLog2e / a->softcap;
    }
  }
  // (every rejection above happens before the first launch: the append below may already write the cache)
  // optional fused append of the step's newest key/value row
  p.new_k = p.new_v = nullptr;
  p.slot_mapping = nullptr;
  p.nk_st = p.nk_sh = p.nv_st = p.nv_sh = 0;
  const bool want_append = a->new_key || a->new_value || a->new_slot_mapping;
  if (want_append) {
    if (!a->new_key || !a->new_value || !a->new_slot_mapping)
      return fail(SB_ERR_INVALID, "sb_swa_decode: new_key, new_value and new_slot_mapping go together");
    if (!a->block_table || a->row_seq)
      return fail(SB_ERR_INVALID, "sb_swa_decode: fused append needs paged mode and one query row per sequence");
    if (((reinterpret_cast<uintptr_t>(a->new_key) | reinterpret_cast<uintptr_t>(a->new_value)) & 15u) ||
        (a->new_key_stride_row * esz) % 16 || (a->new_key_stride_head * esz) % 16 ||
        (a->new_value_stride_row * esz) % 16 || (a->new_value_stride_head * esz) % 16)
      return fail(SB_ERR_INVALID, "sb_swa_decode: new key/value rows must be 16-byte aligned");
    if (mfma && a->phases != 2) {
      p.new_k = (const char *)a->new_key; p.new_v = (const char *)a->new_value;
      p.slot_mapping = a->new_slot_mapping;
      p.nk_st = a->new_key_stride_row * esz; p.nk_sh = a->new_key_stride_head * esz;
      p.nv_st = a->new_value_stride_row * esz; p.nv_sh = a->new_value_stride_head * esz;
    } else if (a->phases != 2) {
      // vector-ALU path: same semantics as two launches
      sb_kv_append_args ap;
      ap.key = a->new_key; ap.value = a->new_value;
      ap.k_cache = const_cast<void *>(a->k_cache); ap.v_cache = const_cast<void *>(a->v_cache);
      ap.slot_mapping = a->new_slot_mapping; ap.num_tokens = a->num_rows;
      ap.num_kv_heads = a->num_kv_heads; ap.head_size = a->head_size; ap.block_size = a->block_size;
      ap.dtype = a->dtype;
      ap.key_stride_token = a->new_key_stride_row; ap.key_stride_head = a->new_key_stride_head;
      ap.value_stride_token = a->new_value_stride_row; ap.value_stride_head = a->new_value_stride_head;
      ap.cache_stride_block = a->kv_stride_block; ap.cache_stride_row = a->kv_stride_row;
      ap.cache_stride_head = a->kv_stride_head; ap.num_blocks = 0; ap.stream = a->stream;
      const int arc = sb_kv_append(&ap);
      if (arc != SB_OK) return arc;
    }
  }
  // (the balanced kernels number the chunks of all rows on one 32-bit axis: a row holds at most its table's
  // or its window's keys)
  int64_t row_chunks_max = (int64_t)1 << 26;
  if (a->block_table) row_chunks_max = std::min<int64_t>(row_chunks_max, a->block_table_stride * (int64_t)a->block_size / 32 + 2);
  if (a->window_left >= 0) row_chunks_max = std::min<int64_t>(row_chunks_max, (int64_t)a->window_left / 32 + 3);
  if (mfma && !int8_kv && n_split > 1 && a->num_rows <= kBalancedMaxRows && (a->flags & SB_DECODE_BALANCED) &&
      a->num_rows * row_chunks_max < ((int64_t)1 << 30))
    p.n_wg = (int)balanced_workgroups(a->num_rows, n_split);
  // On request the fixed split of the matrix-core kernel merges in the same launch (the last wavefront of a
  // row to finish does it), where the arrival counters fit; otherwise the merge kernel follows as usual.
  if ((a->flags & SB_DECODE_MERGE_IN_KERNEL) && mfma && !int8_kv && n_split > 1 && n_split <= 64 && p.n_wg == 0 &&
      a->phases == 0 && ((a->flags >> 4) & 7) <= 1 && a->meta_len == 0 &&
      (a->num_rows + 7) / 8 * 8 * (int64_t)a->num_kv_heads <= kMergeCounters)
    p.merge_counter = (int *)a->workspace;
  // the serving path (paged element cache, one query row per sequence, no key_lo, no meta rows) runs the
  // split as one stream of chunks per wavefront
  const bool stream = mfma && !int8_kv && !(a->flags & SB_DECODE_PER_SEGMENT) && a->block_table && !a->row_seq &&
                      !a->key_lo && a->meta_len == 0 && !p.merge_counter && ((a->flags >> 4) & 7) <= 1 &&
                      (int64_t)a->num_q_heads * a->q_stride_head * esz < (1LL << 31);
  if (a->phases != 2) {
    if (int8_kv) launch_swa_decode_split_i8(a->dtype, a->kv_quant, G, a->num_kv_heads, (unsigned)a->num_rows, (unsigned)n_split, st, p);
    else if (stream)
      launch_swa_decode_stream(a->dtype, G, a->num_kv_heads, (unsigned)a->num_rows, (unsigned)n_split, st, p,
                               (hipEvent_t)a->profile_start_event, (hipEvent_t)a->profile_stop_event);
    else if (mfma) launch_swa_decode_split_mfma(a->dtype, G, a->num_kv_heads, (unsigned)a->num_rows, (unsigned)n_split,
                                           (a->flags >> 4) & 7, st, p, (hipEvent_t)a->profile_start_event,
                                           (hipEvent_t)a->profile_stop_event);
    else {
      const dim3 vgrid((unsigned)a->num_rows, (unsigned)(a->num_kv_heads * p.group_parts), (unsigned)n_split);
      if (a->dtype == SB_BF16) rc = launch_for_group<BF16>(vec_g, vgrid, st, p);
      else if (a->dtype == SB_F16) rc = launch_for_group<F16>(vec_g, vgrid, st, p);
      else rc = launch_for_group<F32>(vec_g, vgrid, st, p);
    }
    if (rc == SB_OK) rc = check_launch("swa_decode_split_kernel");
  }
  if (rc != SB_OK || n_split == 1 || a->phases == 1 || p.merge_counter) return rc;

  const dim3 mgrid((unsigned)(a->num_rows * a->num_q_heads));
  if (p.n_wg > 0 && stream) {
    if (a->dtype == SB_BF16) hipLaunchKernelGGL(swa_decode_merge_rows_kernel<BF16>, mgrid, dim3(128), 0, st, p);
    else hipLaunchKernelGGL(swa_decode_merge_rows_kernel<F16>, mgrid, dim3(128), 0, st, p);
    return check_launch("swa_decode_merge_rows_kernel");
  }
  if (p.n_wg > 0) {
    if (a->dtype == SB_BF16) hipLaunchKernelGGL(swa_decode_merge_balanced_kernel<BF16>, mgrid, dim3(128), 0, st, p);
    else hipLaunchKernelGGL(swa_decode_merge_balanced_kernel<F16>, mgrid, dim3(128), 0, st, p);
    return check_launch("swa_decode_merge_balanced_kernel");
  }
  const dim3 mblock((unsigned)a->head_size);
  if (a->dtype == SB_BF16) hipLaunchKernelGGL(swa_decode_merge_kernel<BF16>, mgrid, mblock, 0, st, p);
  else if (a->dtype == SB_F16) hipLaunchKernelGGL(swa_decode_merge_kernel<F16>, mgrid, mblock, 0, st, p);
  else hipLaunchKernelGGL(swa_decode_merge_kernel<F32>, mgrid, mblock, 0, st, p);
  return check_launch("swa_decode_merge_kernel");
}

// ---- sb_swa_decode_static: the same call, partial results in memory the library itself holds ------
// The split-K partials go into a file-scope device array instead of a caller workspace, so the call
// touches no allocator at all. Every GPU the library runs on holds its own copy of the array (at its
// own address) until the process ends; the array's name is only a host-side handle for
// hipGetSymbolAddress, the address that call returns is what kernels and copies are given.
static __device__ __align__(256) unsigned char scratch[SB_SWA_DECODE_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices];  // per device: address of that device's copy of `scratch`, once looked up
}  // namespace

extern "C" int sb_swa_decode_static(const sb_swa_decode_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_swa_decode_static: null args");
  if (a->num_rows < 0) return fail(SB_ERR_INVALID, "sb_swa_decode_static: negative num_rows");
  if (a->num_rows == 0) return SB_OK;
  int n_split = a->n_split;
  if (n_split < 0) return fail(SB_ERR_INVALID, "sb_swa_decode_static: negative n_split");
  if (n_split == 0)
    n_split = sb_swa_decode_auto_split(a->num_rows, a->num_kv_heads, a->max_seq_len, a->window_left);
  const size_t need = sb_swa_decode_workspace_bytes(a->num_rows, a->num_q_heads, a->head_size, n_split);
  if (need > (size_t)SB_SWA_DECODE_STATIC_SCRATCH_BYTES)
    return fail(SB_ERR_WORKSPACE,
                "sb_swa_decode_static: %lld rows x %d heads in %d splits need %zu bytes of partial results, the "
                "library's own scratch holds %zu (use sb_swa_decode with a workspace, or fewer splits)",
                (long long)a->num_rows, a->num_q_heads, n_split, need, (size_t)SB_SWA_DECODE_STATIC_SCRATCH_BYTES);
  sb_swa_decode_args b = *a;
  b.n_split = n_split;
  b.workspace = nullptr;
  b.workspace_bytes = 0;
  if (need > 0) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "sb_swa_decode_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices)
      return fail(SB_ERR_UNSUPPORTED, "sb_swa_decode_static: device index %d (at most %d devices)", dev, kMaxDevices);
    void *ptr = nullptr;
    {
      std::lock_guard<std::mutex> lock(g_scratch_mu);
      ptr = g_scratch_ptr[dev];
      if (!ptr) {  // first call on this device (must not be under stream capture)
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
          return fail(e != hipSuccess ? (int)e : SB_ERR_INVALID, "sb_swa_decode_static: hipGetSymbolAddress: %s",
                      hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
      }
    }
    b.workspace = ptr;
    b.workspace_bytes = (size_t)SB_SWA_DECODE_STATIC_SCRATCH_BYTES;
  }
  return sb_swa_decode(&b);
}

extern "C" int sb_lse_merge(const sb_lse_merge_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_lse_merge: null args");
  if (a->rows < 0 || a->heads < 0) return fail(SB_ERR_INVALID, "sb_lse_merge: negative size");
  if (a->rows == 0 || a->heads == 0) return SB_OK;
  if (!a->out || !a->lse || !a->block_out || !a->block_lse)
    return fail(SB_ERR_INVALID, "sb_lse_merge: null tensor pointer");
  if (a->head_size <= 0 || a->head_size % 8 != 0)
    return fail(SB_ERR_UNSUPPORTED, "sb_lse_merge: head_size %d must be a positive multiple of 8", a->head_size);
  int esz;
  switch (a->dtype) {
    case SB_BF16:
    case SB_F16: esz = 2; break;
    case SB_F32: esz = 4; break;
    default: return fail(SB_ERR_UNSUPPORTED, "sb_lse_merge: unknown dtype %d", a->dtype);
  }
  const int64_t es[] = {a->out_stride_row, a->out_stride_head, a->block_out_stride_row, a->block_out_stride_head};
  for (int64_t s : es)
    if ((s * esz) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_lse_merge: stride %lld elements is not 16-byte aligned", (long long)s);
  if ((reinterpret_cast<uintptr_t>(a->out) | reinterpret_cast<uintptr_t>(a->block_out)) & 15u)
    return fail(SB_ERR_INVALID, "sb_lse_merge: out/block_out base not 16-byte aligned");
  LseMergeParams p;
  p.out = (char *)a->out; p.lse = a->lse; p.block_out = (const char *)a->block_out; p.block_lse = a->block_lse;
  p.pairs = a->rows * a->heads; p.heads = a->heads; p.vecs = a->head_size / 8;
  p.o_sr = a->out_stride_row; p.o_sh = a->out_stride_head;
  p.b_sr = a->block_out_stride_row; p.b_sh = a->block_out_stride_head;
  const int64_t threads = p.pairs * p.vecs;
  if ((threads + 255) / 256 > 0x7fffffffLL) return fail(SB_ERR_UNSUPPORTED, "sb_lse_merge: too many rows");
  const dim3 grid((unsigned)((threads + 255) / 256));
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == SB_BF16) hipLaunchKernelGGL(lse_merge_kernel<BF16>, grid, dim3(256), 0, st, p);
  else if (a->dtype == SB_F16) hipLaunchKernelGGL(lse_merge_kernel<F16>, grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL(lse_merge_kernel<F32>, grid, dim3(256), 0, st, p);
  return check_launch("lse_merge_kernel");
}
