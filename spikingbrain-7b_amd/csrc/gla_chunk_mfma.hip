// GLA over prompts on the matrix cores: the recurrence S <- diag(exp g) S + k^T v, o = (q*scale) S
// advanced 16 tokens at a time in its exact block form. With B_t = g_1 + .. + g_t (per key dim,
// inside the block) and S_0 the state before the block,
//   o_t  = (q_t * exp(B_t)) S_0 + sum_{s<=t} [(q_t * exp(B_t)) . (k_s * exp(-B_s))] v_s
//   S_16 = diag(exp(B_16)) S_0 + sum_s (k_s * exp(B_16 - B_s))^T v_s
// i.e. per block one [16x16] score product, two products into o and a rank-16 update of the state,
// all v_mfma_f32_16x16x32_bf16 with fp32 accumulation. The reference computes prompts with fla's
// fused_chunk_gla (vllm_hymeta/model_for_7B/gla_attention.py:207-208), the same block mathematics.
//
// One workgroup per (sequence, head), four wavefronts; wavefront w keeps the state columns
// [32w, 32w+32) as 16 accumulator tiles (64 registers) for the whole prompt: the state crosses HBM
// once each way. Per block: all threads turn q, k, g, v into the five LDS operands (gate scan per
// key dim in fp32), one barrier, then each wavefront runs its 30 matrix instructions. LDS is
// double-buffered, so one barrier per block is enough; the loads of the next block are in flight
// during the matrix phase.
//
// Precision: 16 tokens fill half of the instruction's K = 32, and the other half carries a second
// bf16 term: the state update uses k * exp(B_16 - B_s) as hi + lo, so the state keeps fp32-level
// accuracy (decay and accumulation are fp32; v is bf16 as given), and the scores enter o = A v as
// hi + lo as well (their 16 signed products per row do not average out a 2^-9 rounding). The rest of
// the output path rounds its operands (q*exp(B), k*exp(-B), S_0) to bf16 like any bf16 GEMM.
// exp(-B_s) grows with the gates inside one block only: 16 * max|g| stays far below the fp32/bf16
// exponent range for any log-sigmoid gate; the exponent is clamped at 80 as a guard.
//
// Tile row order: accumulator tile rt of the state holds rows 32*(rt/2) + 8*(m/4) + 4*(rt%2) + m%4
// (m = tile row), so that the 8 consecutive rows a lane needs as the B operand of q S_0 are exactly
// the rows it already holds in tiles 2*st and 2*st+1: no cross-lane movement between the update
// and the next block's read of the state.
#include "common.h"
#include "mfma_util.h"

namespace {

using namespace sb;

struct GlaChunkParams {
  const uint16_t *q, *k, *v;  // bf16
  const void *g;
  void *state;
  uint16_t *out;
  const int32_t *slot_idx;
  const int32_t *cu;
  int H, T;
  float scale;
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, g_sb, g_sh, g_st, o_sb, o_sh, o_st;
  int64_t s_slot, s_head;
  // Shared states: G query heads per head of k, v, g and state; head index hh of this launch (H of them)
  // stands for state head hh / jn and query head (hh / jn) * G + j0 + hh % jn; write_state: store the
  // final state. One state per head: G = jn = 1, j0 = 0, write_state = 1.
  int G, jn, j0, write_state;
};

constexpr int kCB = 16;      // tokens per block
constexpr int kRow = 136;    // elements per row of the [16][128] operands (272 B: 16-byte aligned, banks spread)
constexpr int kTRow = 24;    // elements per row of the transposed [128][16] operands (48 B)
constexpr float kMaxExp = 80.f;

struct Stage {
  uint16_t qs[kCB][kRow];       // q * exp(B_t) * scale
  uint16_t ks[kCB][kRow];       // k * exp(-B_t)
  uint16_t kh_hi[128][kTRow];   // (k * exp(B_16 - B_t))^T, high part
  uint16_t kh_lo[128][kTRow];   // low part
  uint16_t vt[128][kTRow];      // v^T
  float dec[128];               // exp(B_16)
};

template <int GDT>
__device__ __forceinline__ float load_gate(const void *p, int64_t i) {
  if constexpr (GDT == SB_F32) return reinterpret_cast<const float *>(p)[i];
  else if constexpr (GDT == SB_BF16) return __uint_as_float((uint32_t) reinterpret_cast<const uint16_t *>(p)[i] << 16);
  else return (float)reinterpret_cast<const _Float16 *>(p)[i];
}

__device__ __forceinline__ float bf16_to_f32(uint16_t x) { return __uint_as_float((uint32_t)x << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }  // v_cvt_pk_bf16_f32

template <bool kStateF32, int GDT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gla_chunk_kernel(const GlaChunkParams p) {
  const int b = blockIdx.x / p.H;
  const int hh = blockIdx.x - b * p.H;
  const int hk = hh / p.jn;
  const int h = hk * p.G + p.j0 + (hh - hk * p.jn);
  const int64_t slot = p.slot_idx ? (int64_t)p.slot_idx[b] : (int64_t)b;
  if (slot < 0) return;
  int T = p.T;
  int64_t qo, ko, vo, go, oo;
  if (p.cu) {
    const int64_t t0 = p.cu[b];
    T = p.cu[b + 1] - (int)t0;
    qo = t0 * p.q_st; ko = t0 * p.k_st; vo = t0 * p.v_st; go = t0 * p.g_st; oo = t0 * p.o_st;
  } else {
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; go = b * p.g_sb; oo = b * p.o_sb;
  }
  if (T <= 0) return;
  qo += h * p.q_sh; ko += hk * p.k_sh; vo += hk * p.v_sh; go += hk * p.g_sh; oo += h * p.o_sh;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int g = lane >> 4, c = lane & 15;
  const int d = tid & 127;        // key dim (gate scan) / value column (transpose) of this thread
  const bool second = tid >= 128;  // threads 0..127: q and k operands; 128..255: k-hat and v

  __shared__ __attribute__((aligned(16))) Stage stage[2];

  // ---- state: 8 row tiles x 2 column tiles of this wavefront's 32 columns -------------------------
  char *sbase = reinterpret_cast<char *>(p.state) + (slot * p.s_slot + (int64_t)hk * p.s_head) * (kStateF32 ? 4 : 2);
  f32x4_t S[8][2];
  auto state_index = [&](int rt, int nt, int i) {
    return (32 * (rt >> 1) + 8 * g + 4 * (rt & 1) + i) * 128 + 32 * w + 16 * nt + c;
  };
#pragma unroll
  for (int rt = 0; rt < 8; ++rt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int idx = state_index(rt, nt, i);
        S[rt][nt][i] = kStateF32 ? reinterpret_cast<const float *>(sbase)[idx]
                                 : bf16_to_f32(reinterpret_cast<const uint16_t *>(sbase)[idx]);
      }

  // ---- block inputs in registers: gates and k for every thread, q (first half) or v (second half) ----
  float rg[kCB];
  uint16_t rk[kCB], rx[kCB];
  // per-thread column pointers once; a token adds a wave-uniform multiple of the row stride
  const char *gp = reinterpret_cast<const char *>(p.g) + (go + d) * (GDT == SB_F32 ? 4 : 2);
  const uint16_t *kp = p.k + ko + d;
  const uint16_t *xp = second ? p.v + vo + d : p.q + qo + d;
  const int64_t xs = second ? p.v_st : p.q_st;
  auto fetch = [&](int t0) {
    const int last = T - 1 - t0;  // rows past the end re-read the last token; they are zeroed when used
    if (last >= kCB - 1) {
#pragma unroll
      for (int t = 0; t < kCB; ++t) {
        rg[t] = load_gate<GDT>(gp, (t0 + t) * p.g_st);
        rk[t] = kp[(t0 + t) * p.k_st];
        rx[t] = xp[(t0 + t) * xs];
      }
    } else {
#pragma unroll
      for (int t = 0; t < kCB; ++t) {
        const int64_t tt = t0 + min(t, last);
        rg[t] = load_gate<GDT>(gp, tt * p.g_st);
        rk[t] = kp[tt * p.k_st];
        rx[t] = xp[tt * xs];
      }
    }
  };

  const int n_blocks = (T + kCB - 1) / kCB;
  fetch(0);
  for (int blk = 0; blk < n_blocks; ++blk) {
    Stage &st = stage[blk & 1];
    const int t0 = blk * kCB;
    // ---- operands of this block ------------------------------------------------------------------
    {
      float B[kCB];
      float run = 0.f;
#pragma unroll
      for (int t = 0; t < kCB; ++t) {
        run += (t0 + t < T) ? rg[t] : 0.f;
        B[t] = run;
      }
      if (!second) {
#pragma unroll
        for (int t = 0; t < kCB; ++t) {
          const bool live = t0 + t < T;
          const float qv = live ? bf16_to_f32(rx[t]) : 0.f, kv = live ? bf16_to_f32(rk[t]) : 0.f;
          st.qs[t][d] = f32_to_bf16(qv * __expf(B[t]) * p.scale);
          st.ks[t][d] = f32_to_bf16(kv * __expf(fminf(-B[t], kMaxExp)));
        }
        st.dec[d] = __expf(run);
      } else {
        uint32_t hi[kCB / 2], lo[kCB / 2], vv[kCB / 2];
#pragma unroll
        for (int t = 0; t < kCB; t += 2) {
          float x[2];
          uint16_t xh[2], xl[2], xv[2];
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const bool live = t0 + t + u < T;
            x[u] = live ? bf16_to_f32(rk[t + u]) * __expf(run - B[t + u]) : 0.f;
            xh[u] = f32_to_bf16(x[u]);
            xl[u] = f32_to_bf16(x[u] - bf16_to_f32(xh[u]));
            xv[u] = live ? rx[t + u] : (uint16_t)0;
          }
          hi[t / 2] = xh[0] | ((uint32_t)xh[1] << 16);
          lo[t / 2] = xl[0] | ((uint32_t)xl[1] << 16);
          vv[t / 2] = xv[0] | ((uint32_t)xv[1] << 16);
        }
        reinterpret_cast<uint4 *>(&st.kh_hi[d][0])[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        reinterpret_cast<uint4 *>(&st.kh_hi[d][0])[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
        reinterpret_cast<uint4 *>(&st.kh_lo[d][0])[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        reinterpret_cast<uint4 *>(&st.kh_lo[d][0])[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
        reinterpret_cast<uint4 *>(&st.vt[d][0])[0] = make_uint4(vv[0], vv[1], vv[2], vv[3]);
        reinterpret_cast<uint4 *>(&st.vt[d][0])[1] = make_uint4(vv[4], vv[5], vv[6], vv[7]);
      }
    }
    if (blk + 1 < n_blocks) fetch(t0 + kCB);  // in flight during the matrix phase
    __syncthreads();

    // ---- scores (transposed): at[i] = A[t = c][s = 4g + i], zero above the diagonal ------------------
    uint4 qa[4];
    f32x4_t at = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
      qa[s4] = *reinterpret_cast<const uint4 *>(&st.qs[c][32 * s4 + 8 * g]);
      const uint4 ka = *reinterpret_cast<const uint4 *>(&st.ks[c][32 * s4 + 8 * g]);
      at = Mma<BF16>::run(ka, qa[s4], at);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (4 * g + i > c) at[i] = 0.f;
    // as the A operand of o = A v: row t = c, k index 8g + j <-> s = 4g + j for j < 4; the scores go in
    // as two bf16 terms (hi in k index 0..3, lo in 4..7, against v repeated), so that the 16 signed
    // products of a row are summed from scores good to 16 bits
    float at_lo[4];
    uint16_t at_hi[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      at_hi[i] = f32_to_bf16(at[i]);
      at_lo[i] = at[i] - bf16_to_f32(at_hi[i]);
    }
    const uint4 pa = make_uint4(at_hi[0] | ((uint32_t)at_hi[1] << 16), at_hi[2] | ((uint32_t)at_hi[3] << 16),
                                Mma<BF16>::pack(at_lo[0], at_lo[1]), Mma<BF16>::pack(at_lo[2], at_lo[3]));

    // v as the B operand of both products: v[s = 4g + j][col] at k index j and again at 4 + j, so
    // that the A operands can carry a high term in k index 0..3 and a low term in 4..7 (16 tokens
    // fill only half of the instruction's K = 32)
    uint4 vb[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const uint2 x = *reinterpret_cast<const uint2 *>(&st.vt[32 * w + 16 * nt + c][4 * g]);
      vb[nt] = make_uint4(x.x, x.y, x.x, x.y);
    }

    // ---- o^T = v^T A^T + S_0^T (q exp B)^T: lane (g, c) ends up with token c, columns 4g..4g+3 of each tile:
    // one 8-byte store per tile (the operand registers are the same either way round: a lane holds
    // index c of the tile's outer dimension and 8g..8g+7 of the contraction in both operands)
    f32x4_t o[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      o[nt] = Mma<BF16>::run(vb[nt], pa, f32x4_t{0.f, 0.f, 0.f, 0.f});
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const f32x4_t &a = S[2 * s4][nt], &bb = S[2 * s4 + 1][nt];  // rows 32 s4 + 8g + {0..3}, {4..7}
        const uint4 sb16 = make_uint4(Mma<BF16>::pack(a[0], a[1]), Mma<BF16>::pack(a[2], a[3]),
                                      Mma<BF16>::pack(bb[0], bb[1]), Mma<BF16>::pack(bb[2], bb[3]));
        o[nt] = Mma<BF16>::run(sb16, qa[s4], o[nt]);
      }
    }
    if (t0 + c < T) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
        *reinterpret_cast<uint2 *>(p.out + oo + (int64_t)(t0 + c) * p.o_st + 32 * w + 16 * nt + 4 * g) =
            make_uint2(Mma<BF16>::pack(o[nt][0], o[nt][1]), Mma<BF16>::pack(o[nt][2], o[nt][3]));
    }

    // ---- S <- diag(exp B_16) S + k-hat^T v ------------------------------------------------------------
#pragma unroll
    for (int rt = 0; rt < 8; ++rt) {
      const float4 dc = *reinterpret_cast<const float4 *>(&st.dec[32 * (rt >> 1) + 8 * g + 4 * (rt & 1)]);
      const int row = 32 * (rt >> 1) + 8 * (c >> 2) + 4 * (rt & 1) + (c & 3);
      const uint2 h2 = *reinterpret_cast<const uint2 *>(&st.kh_hi[row][4 * g]);
      const uint2 l2 = *reinterpret_cast<const uint2 *>(&st.kh_lo[row][4 * g]);
      const uint4 ka = make_uint4(h2.x, h2.y, l2.x, l2.y);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        f32x4_t s = S[rt][nt];
        s[0] *= dc.x; s[1] *= dc.y; s[2] *= dc.z; s[3] *= dc.w;
        S[rt][nt] = Mma<BF16>::run(ka, vb[nt], s);
      }
    }
  }

  if (!p.write_state) return;
#pragma unroll
  for (int rt = 0; rt < 8; ++rt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int idx = state_index(rt, nt, i);
        if (kStateF32) reinterpret_cast<float *>(sbase)[idx] = S[rt][nt][i];
        else reinterpret_cast<uint16_t *>(sbase)[idx] = f32_to_bf16(S[rt][nt][i]);
      }
}

}  // namespace

namespace sb_host {

// Launch for bf16 q/k/v/out; g of any built type. Grid: one workgroup per (row, head).
void launch_gla_chunk(const sb_gla_recurrent_args *a, int64_t groups, int heads, int G, int jn, int j0, int write_state) {
  GlaChunkParams p;
  p.q = (const uint16_t *)a->q; p.k = (const uint16_t *)a->k; p.v = (const uint16_t *)a->v; p.g = a->g;
  p.state = a->state; p.out = (uint16_t *)a->out; p.slot_idx = a->slot_idx; p.cu = a->cu_seqlens;
  p.H = heads; p.T = a->seq_len; p.scale = a->scale;
  p.G = G; p.jn = jn; p.j0 = j0; p.write_state = write_state;
  p.q_sb = a->q_stride_b; p.q_sh = a->q_stride_h; p.q_st = a->q_stride_t;
  p.k_sb = a->k_stride_b; p.k_sh = a->k_stride_h; p.k_st = a->k_stride_t;
  p.v_sb = a->v_stride_b; p.v_sh = a->v_stride_h; p.v_st = a->v_stride_t;
  p.g_sb = a->g_stride_b; p.g_sh = a->g_stride_h; p.g_st = a->g_stride_t;
  p.o_sb = a->out_stride_b; p.o_sh = a->out_stride_h; p.o_st = a->out_stride_t;
  p.s_slot = a->state_stride_slot; p.s_head = a->state_stride_head;
  const dim3 grid((unsigned)groups), block(256);
  hipStream_t st = (hipStream_t)a->stream;
#define SB_LAUNCH(F32S, GDT) hipLaunchKernelGGL((gla_chunk_kernel<F32S, GDT>), grid, block, 0, st, p)
  if (a->state_dtype == SB_F32) {
    if (a->g_dtype == SB_F32) SB_LAUNCH(true, SB_F32);
    else if (a->g_dtype == SB_BF16) SB_LAUNCH(true, SB_BF16);
    else SB_LAUNCH(true, SB_F16);
  } else {
    if (a->g_dtype == SB_F32) SB_LAUNCH(false, SB_F32);
    else if (a->g_dtype == SB_BF16) SB_LAUNCH(false, SB_BF16);
    else SB_LAUNCH(false, SB_F16);
  }
#undef SB_LAUNCH
}

}  // namespace sb_host
