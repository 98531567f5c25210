// GLA over prompts on the matrix cores: the recurrence S <- diag(exp g) S + k^T v, o = (q*scale) S
// advanced 16 tokens at a time in its exact block form. With B_t = g_1 + .. + g_t (per key dim,
// inside the block) and S_0 the state before the block,
//   o_t  = (q_t * exp(B_t)) S_0 + sum_{s<=t} [(q_t * exp(B_t)) . (k_s * exp(-B_s))] v_s
//   S_16 = diag(exp(B_16)) S_0 + sum_s (k_s * exp(B_16 - B_s))^T v_s
// i.e. per block one [16x16] score product, two products into o and a rank-16 update of the state,
// all v_mfma_f32_16x16x32_bf16 with fp32 accumulation.
// The decay of the state is applied every SECOND block: in between the registers hold S' = diag(exp(-L)) S,
// L = the log-decay of the block just done, and the operands of the next block carry L in their exponents,
//   o_t = (q_t * exp(B_t + L)) S' + intra-block term,   S' <- S' + (k_s * exp(-(B_s + L)))^T v_s,
// after which S = diag(exp(L + B_16)) S' is formed. This halves the multiplies on the 64 state registers,
// and k * exp(-(B_s + L)) serves both as the score operand and, transposed, as the state-update operand. The reference computes prompts with fla's
// fused_chunk_gla (vllm_hymeta/model_for_7B/gla_attention.py:207-208), the same block mathematics.
//
// One workgroup per (sequence, head), four wavefronts; wavefront w keeps the state columns
// [32w, 32w+32) as 16 accumulator tiles (64 registers) for the whole prompt: the state crosses HBM
// once each way. Per block: thread (dim group r = tid / 16, token t = tid % 16) loads 8 consecutive dims of
// its token's q, k, v (16 bytes each) and gate, five or four 16-byte loads instead of 48 two- and
// four-byte ones (the vector memory pipe takes a wave's load at a fixed rate whatever its width); the
// 16 tokens of a dim sit in the 16 lanes of a DPP row, so the gate scan over tokens is four row-shift
// adds per dim. The threads turn their pieces into the four LDS operands, one barrier, then each
// wavefront runs its 30 matrix instructions. LDS is double-buffered, so one barrier per block is
// enough, and a wavefront prepares block n + 1 in the same stretch of code as it multiplies block n.
//
// Precision: 16 tokens fill half of the instruction's K = 32, and the other half carries a second
// bf16 term: the state update uses k * exp(B_16 - B_s) as hi + lo, so the state keeps fp32-level
// accuracy (decay and accumulation are fp32; v is bf16 as given), and the scores enter o = A v as
// hi + lo as well (their 16 signed products per row do not average out a 2^-9 rounding). The rest of
// the output path rounds its operands (q*exp(B), k*exp(-B), S_0) to bf16 like any bf16 GEMM.
// exp(-(B_s + L)) grows with the gates of at most two blocks: 32 * max|g| stays far below the fp32/bf16
// exponent range for any log-sigmoid gate (|g| up to 2.5 per token, sustained); the exponent is clamped at
// 80 as a guard. A wavefront whose gates reach the clamp in a pair of blocks (results then under-weight
// near-diagonal terms) adds one to a device counter that sb_gla_gate_range_hits reads.
//
// Tile row order: accumulator tile rt of the state holds rows 32*(rt/2) + 8*(m/4) + 4*(rt%2) + m%4
// (m = tile row), so that the 8 consecutive rows a lane needs as the B operand of q S_0 are exactly
// the rows it already holds in tiles 2*st and 2*st+1: no cross-lane movement between the update
// and the next block's read of the state.
#include <mutex>

#include "common.h"
#include "mfma_util.h"

// Events of gla_chunk_kernel meeting gates beyond the block form's range (one per wavefront and pair of blocks
// concerned) since the counter was last cleared; one copy per GPU (the name is only the host's handle for
// hipGetSymbolAddress).
static __device__ unsigned int gla_range_hits;

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
  unsigned int *range_hits;  // device counter of (wavefront, pair of blocks) events whose gates reached the exponent clamp
};

constexpr int kCB = 16;      // tokens per block
#ifndef SB_GLA_ROW
#define SB_GLA_ROW 152
#endif
constexpr int kRow = SB_GLA_ROW;    // elements per row of the [16 tokens][128] LDS operands (304 B = 76 dwords: the 16-byte
                             // stores and loads of 16 rows and the transposing loads of 4 rows spread over the banks)
constexpr float kMaxExp = 80.f;

// All operands are stored token-major, one 16-byte store per thread each. The state update and the output
// product contract over tokens and need [dim][token] operands: those are read with the transposing LDS load
// (ds_read_b64_tr_b16), no transposed copy is ever written.
struct Stage {
  uint16_t qs[kCB][kRow];  // q * exp(B_t + L) * scale
  uint16_t ks[kCB][kRow];  // k * exp(-(B_t + L)) rounded to bf16: score operand, and high part of the state-update operand
  uint16_t kl[kCB][kRow];  // what the rounding left: low part of the state-update operand
  uint16_t vs[kCB][kRow];  // v as loaded
  float dec[128];          // exp(L + B_16) (second block of a pair), L + B_16 in log2 units (first block)
};

// ds_read_b64_tr_b16: in every group of 16 lanes, lane i names 8 bytes (4 elements) of LDS, "row i"; lane l
// receives element l % 4 of rows l / 4, l / 4 + 4, l / 4 + 8, l / 4 + 12 (checked on the GPU). With row
// i = (token t0 + i / 4, dims f(i % 4) .. + 3), lane l gets dim f(l / 4) + l % 4 of tokens t0 .. t0 + 3.
__device__ __forceinline__ uint2 load_transposed(const uint16_t *row) {
  typedef short v4s __attribute__((ext_vector_type(4)));
  const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)row);
  return __builtin_bit_cast(uint2, v);
}

// Loads through buffer descriptors: the descriptor holds a block's first row (wave-uniform, scalar registers),
// the thread's token row and column are a 32-bit vector offset that is the same for every block: no vector
// arithmetic per load.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_from(const char *first_row) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(first_row), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ uint4 load16(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
// x of the lane `shift` places down the row of 16 lanes, 0 where the row has no such lane
template <int kShift>
__device__ __forceinline__ float row_shr(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x110 + kShift, 0xf, 0xf, true));
}

__device__ __forceinline__ float bf16_to_f32(uint16_t x) { return __uint_as_float((uint32_t)x << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }  // v_cvt_pk_bf16_f32

// kCheck: report gates beyond the block form's range (SB_GLA_CHECK_GATES); a build of its own, because even this
// little extra work shifts the register allocation of a kernel that runs at the edge of its budget (0-4 % slower).
template <bool kStateF32, int GDT, bool kCheck>
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
  const int r = tid >> 4;          // dims 8r .. 8r+7 of token c: this thread's piece of a block's inputs

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

  // ---- block inputs in registers: 8 dims of one token's q, k, v (bf16) and gate ---------------------------
  constexpr int kGateBytes = GDT == SB_F32 ? 4 : 2;
  const char *gb = reinterpret_cast<const char *>(p.g) + go * kGateBytes;
  const char *qb = reinterpret_cast<const char *>(p.q + qo), *kb = reinterpret_cast<const char *>(p.k + ko),
             *vb_ = reinterpret_cast<const char *>(p.v + vo);
  const int64_t g_row = p.g_st * kGateBytes, q_row = p.q_st * 2, k_row = p.k_st * 2, v_row = p.v_st * 2, o_row = p.o_st * 2;
  struct BlockIn {
    uint4 q, k, v;
    uint4 g[kGateBytes / 2];  // fp32: dims 8r..8r+3, 8r+4..8r+7; 16-bit: all 8
  };
  auto fetch = [&](int t0, BlockIn &in) {
    const int tok = min(c, T - 1 - t0);  // rows past the end re-read the last token; prepare() zeroes them
    in.q = load16(rows_from(qb + t0 * q_row), tok * (int)q_row + r * 16);
    in.k = load16(rows_from(kb + t0 * k_row), tok * (int)k_row + r * 16);
    in.v = load16(rows_from(vb_ + t0 * v_row), tok * (int)v_row + r * 16);
    const __amdgpu_buffer_rsrc_t gr = rows_from(gb + t0 * g_row);
#pragma unroll
    for (int j = 0; j < kGateBytes / 2; ++j) in.g[j] = load16(gr, tok * (int)g_row + r * 8 * kGateBytes + 16 * j);
  };

  // ---- the four LDS operands of one block. Gates in log2 units (bare v_exp afterwards); a token past the
  // end of the prompt is a token with g = 0, q = k = v = 0 ------------------------------------------------
  auto fix_tail = [&](BlockIn &in, int t0) {
    if (t0 + kCB > T && t0 + c >= T) {
      in.q = in.k = in.v = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
      for (int j = 0; j < kGateBytes / 2; ++j) in.g[j] = make_uint4(0u, 0u, 0u, 0u);
    }
  };
  // kSecond = false: first block of a pair (state undecayed on entry: L = 0); leaves L = its total log-decay
  // in `carry` and, for the case that the prompt ends here, in st.dec (log2 units).
  // kSecond = true: exponents carry L; st.dec = exp(L + B_16), the decay multiply() applies afterwards.
  float carry[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) carry[i] = 0.f;
  auto prepare = [&](const BlockIn &in, Stage &st, auto second_tag) {
    constexpr bool kSecond = decltype(second_tag)::value;
    const uint4 rq = in.q, rk = in.k, rv = in.v;
    float B[8], tot[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float x;
      if constexpr (GDT == SB_F32) x = __uint_as_float(word(in.g[i >> 2], i & 3));
      else if constexpr (GDT == SB_BF16) x = (i & 1) ? bf16_hi(word(in.g[0], i >> 1)) : bf16_lo(word(in.g[0], i >> 1));
      else x = (i & 1) ? f16_hi(word(in.g[0], i >> 1)) : f16_lo(word(in.g[0], i >> 1));
      x *= kLog2e;
      // inclusive scan over the 16 tokens = the 16 lanes of this row
      x += row_shr<1>(x);
      x += row_shr<2>(x);
      x += row_shr<4>(x);
      x += row_shr<8>(x);
      if constexpr (kSecond) x += carry[i];
      B[i] = x;
      tot[i] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane | 15) << 2, __builtin_bit_cast(int, x)));
    }
    // Gate range: the largest exponent formed inside a pair of blocks is minus its total log-decay. Checked where
    // the pair ends, and reported on the spot (a flag carried through the loop costs this kernel 6 %: it runs at
    // the edge of its register budget).
    if constexpr (kSecond && kCheck) {
      const float worst = fminf(fminf(fminf(tot[0], tot[1]), fminf(tot[2], tot[3])), fminf(fminf(tot[4], tot[5]), fminf(tot[6], tot[7])));
      if (__builtin_amdgcn_ballot_w64(worst < -kMaxExp * kLog2e) != 0 && lane == 0) atomicAdd(p.range_hits, 1u);
    }
    float qf[8], kf[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      qf[2 * i] = bf16_lo(word(rq, i));
      qf[2 * i + 1] = bf16_hi(word(rq, i));
      kf[2 * i] = bf16_lo(word(rk, i));
      kf[2 * i + 1] = bf16_hi(word(rk, i));
    }
    uint32_t qs[4], ks[4], kl[4];
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      qs[i / 2] = Mma<BF16>::pack(qf[i] * p.scale * fast_exp2(B[i]), qf[i + 1] * p.scale * fast_exp2(B[i + 1]));
      const float x0 = kf[i] * fast_exp2(fminf(-B[i], kMaxExp * kLog2e)), x1 = kf[i + 1] * fast_exp2(fminf(-B[i + 1], kMaxExp * kLog2e));
      // the rounded value is the score operand and the high part of the state-update operand
      const uint32_t h = Mma<BF16>::pack(x0, x1);
      const uint32_t l = Mma<BF16>::pack(x0 - __uint_as_float(h << 16), x1 - __uint_as_float(h & 0xffff0000u));
      ks[i / 2] = h;
      kl[i / 2] = l;
    }
    *reinterpret_cast<uint4 *>(&st.qs[c][8 * r]) = make_uint4(qs[0], qs[1], qs[2], qs[3]);
    *reinterpret_cast<uint4 *>(&st.ks[c][8 * r]) = make_uint4(ks[0], ks[1], ks[2], ks[3]);
    *reinterpret_cast<uint4 *>(&st.kl[c][8 * r]) = make_uint4(kl[0], kl[1], kl[2], kl[3]);
    *reinterpret_cast<uint4 *>(&st.vs[c][8 * r]) = rv;
    // (every lane of the row holds the same totals and stores them to the same address: no branch here)
    if constexpr (kSecond) {
      *reinterpret_cast<float4 *>(&st.dec[8 * r]) = make_float4(fast_exp2(tot[0]), fast_exp2(tot[1]), fast_exp2(tot[2]), fast_exp2(tot[3]));
      *reinterpret_cast<float4 *>(&st.dec[8 * r + 4]) = make_float4(fast_exp2(tot[4]), fast_exp2(tot[5]), fast_exp2(tot[6]), fast_exp2(tot[7]));
    } else {
      *reinterpret_cast<float4 *>(&st.dec[8 * r]) = make_float4(tot[0], tot[1], tot[2], tot[3]);
      *reinterpret_cast<float4 *>(&st.dec[8 * r + 4]) = make_float4(tot[4], tot[5], tot[6], tot[7]);
#pragma unroll
      for (int i = 0; i < 8; ++i) carry[i] = tot[i];
    }
  };

  // ---- the 30 matrix instructions of one block on this wavefront's 32 state columns ---------------------
  auto multiply = [&](int t0, const Stage &st, auto second_tag) {
    constexpr bool kSecond = decltype(second_tag)::value;
    // scores (transposed): at[i] = A[t = c][s = 4g + i], zero above the diagonal
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
    const uint32_t h01 = Mma<BF16>::pack(at[0], at[1]), h23 = Mma<BF16>::pack(at[2], at[3]);
    const uint4 pa = make_uint4(h01, h23,
                                Mma<BF16>::pack(at[0] - __uint_as_float(h01 << 16), at[1] - __uint_as_float(h01 & 0xffff0000u)),
                                Mma<BF16>::pack(at[2] - __uint_as_float(h23 << 16), at[3] - __uint_as_float(h23 & 0xffff0000u)));

    // v as the B operand of both products: v[s = 4g + j][col] at k index j and again at 4 + j, so
    // that the A operands can carry a high term in k index 0..3 and a low term in 4..7 (16 tokens
    // fill only half of the instruction's K = 32)
    uint4 vb[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const uint2 x = load_transposed(&st.vs[4 * g + (c >> 2)][32 * w + 16 * nt + 4 * (c & 3)]);
      vb[nt] = make_uint4(x.x, x.y, x.x, x.y);
    }

    // o^T = v^T A^T + S_0^T (q exp B)^T: lane (g, c) ends up with token c, columns 4g..4g+3 of each tile:
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
    {  // rows past the end of the prompt fall outside the descriptor and are dropped: no branch in this code
      const __amdgpu_buffer_rsrc_t orows = __builtin_amdgcn_make_buffer_rsrc(
          reinterpret_cast<char *>(p.out + oo) + t0 * o_row, 0, min(kCB, T - t0) * (int)o_row, 0x00020000);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
        u32x2_t val;
        val.x = Mma<BF16>::pack(o[nt][0], o[nt][1]);
        val.y = Mma<BF16>::pack(o[nt][2], o[nt][3]);
        __builtin_amdgcn_raw_buffer_store_b64(val, orows, c * (int)o_row + (32 * w + 16 * nt + 4 * g) * 2, 0, 0);
      }
    }

    // S' <- S' + k-hat^T v, and after the second block of a pair S <- diag(exp(L + B_16)) S'
#pragma unroll
    for (int rt = 0; rt < 8; ++rt) {
      // this lane's operand row is state row 32 (rt / 2) + 8 (c / 4) + 4 (rt % 2) + c % 4: f(j) = 32 (rt / 2) + 8 j + 4 (rt % 2)
      const int tok = 4 * g + (c >> 2), dims = 32 * (rt >> 1) + 8 * (c & 3) + 4 * (rt & 1);
      const uint2 h2 = load_transposed(&st.ks[tok][dims]);
      const uint2 l2 = load_transposed(&st.kl[tok][dims]);
      const uint4 ka = make_uint4(h2.x, h2.y, l2.x, l2.y);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) S[rt][nt] = Mma<BF16>::run(ka, vb[nt], S[rt][nt]);
      if constexpr (kSecond) {
        const float4 dc = *reinterpret_cast<const float4 *>(&st.dec[32 * (rt >> 1) + 8 * g + 4 * (rt & 1)]);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          S[rt][nt][0] *= dc.x; S[rt][nt][1] *= dc.y; S[rt][nt][2] *= dc.z; S[rt][nt][3] *= dc.w;
        }
      }
    }
  };

  // ---- block loop. An iteration runs the matrix instructions of block blk and turns the inputs of block
  // blk + 1 into the other LDS stage, then fetches the inputs of block blk + 2 into the registers just used; a
  // fetch past the last block re-reads it, and the block after the last is prepared as 16 dead tokens (never
  // multiplied). One barrier per block: what an iteration writes was last read one iteration before the
  // barrier it follows. Blocks go in pairs (first, second); a prompt that ends on a first block leaves
  // S' = diag(exp(-L)) S in the registers, put right after the loop.
  const int n_blocks = (T + kCB - 1) / kCB;
  const std::false_type kFirst{};
  const std::true_type kSecond{};
  BlockIn in;
  fetch(0, in);
  fix_tail(in, 0);
  prepare(in, stage[0], kFirst);
  fetch(min(1, n_blocks - 1) * kCB, in);
  int blk = 0;
  for (; blk + 1 < n_blocks; blk += 2) {
    __syncthreads();
    fix_tail(in, (blk + 1) * kCB);
    multiply(blk * kCB, stage[0], kFirst);
    prepare(in, stage[1], kSecond);
    fetch(min(blk + 2, n_blocks - 1) * kCB, in);
    __syncthreads();
    fix_tail(in, (blk + 2) * kCB);
    multiply((blk + 1) * kCB, stage[1], kSecond);
    prepare(in, stage[0], kFirst);
    fetch(min(blk + 3, n_blocks - 1) * kCB, in);
  }
  if (blk < n_blocks) {
    __syncthreads();
    multiply(blk * kCB, stage[0], kFirst);
    float worst = 0.f;  // (a last block without a partner: its own total is the exponent range it used)
#pragma unroll
    for (int rt = 0; rt < 8; ++rt) {
      const float4 dc = *reinterpret_cast<const float4 *>(&stage[0].dec[32 * (rt >> 1) + 8 * g + 4 * (rt & 1)]);
      if constexpr (kCheck) worst = fminf(worst, fminf(fminf(dc.x, dc.y), fminf(dc.z, dc.w)));
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        S[rt][nt][0] *= fast_exp2(dc.x); S[rt][nt][1] *= fast_exp2(dc.y);
        S[rt][nt][2] *= fast_exp2(dc.z); S[rt][nt][3] *= fast_exp2(dc.w);
      }
    }
    if constexpr (kCheck)
      if (__builtin_amdgcn_ballot_w64(worst < -kMaxExp * kLog2e) != 0 && tid == 0) atomicAdd(p.range_hits, 1u);
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


// ---- one pass for a whole GQA group (shared states) -----------------------------------------------------------
// One workgroup per (sequence, state head): the state is advanced ONCE per block and the outputs of all G query
// heads of the group are formed against it, instead of one workgroup per query head each carrying the whole
// recurrence (G - 1 of them only for their outputs). Per head the arithmetic and its order are those of
// gla_chunk_kernel (same operands, same matrix instructions in the same sequence), so the results are the same
// bits. The q operands of the G heads sit side by side in LDS; k-hat, v and the decays are prepared once.
constexpr int kMaxGroup = 8;

struct GroupStage {
  uint16_t qs[kMaxGroup][kCB][kRow];
  uint16_t ks[kCB][kRow];
  uint16_t kl[kCB][kRow];
  uint16_t vs[kCB][kRow];
  float dec[128];
};

template <bool kStateF32, int GDT>
__global__ __launch_bounds__(256) void gla_chunk_group_kernel(const GlaChunkParams p) {
  const int b = blockIdx.x / p.H;   // p.H: state heads here
  const int hk = blockIdx.x - b * p.H;
  const int G = p.G;
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
  qo += (int64_t)hk * G * p.q_sh; ko += hk * p.k_sh; vo += hk * p.v_sh; go += hk * p.g_sh; oo += (int64_t)hk * G * p.o_sh;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int g = lane >> 4, c = lane & 15;
  const int r = tid >> 4;

  extern __shared__ __attribute__((aligned(16))) char group_smem[];
  GroupStage *const stage = reinterpret_cast<GroupStage *>(group_smem);

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

  constexpr int kGateBytes = GDT == SB_F32 ? 4 : 2;
  const char *gb = reinterpret_cast<const char *>(p.g) + go * kGateBytes;
  const char *qb = reinterpret_cast<const char *>(p.q + qo), *kb = reinterpret_cast<const char *>(p.k + ko),
             *vb_ = reinterpret_cast<const char *>(p.v + vo);
  const int64_t g_row = p.g_st * kGateBytes, q_row = p.q_st * 2, k_row = p.k_st * 2, v_row = p.v_st * 2, o_row = p.o_st * 2;
  const int q_head = (int)(p.q_sh * 2), o_head = (int)(p.o_sh * 2);  // bytes between the group's heads (host-checked to fit)
  struct BlockIn {
    uint4 q[kMaxGroup], k, v;
    uint4 g[kGateBytes / 2];
  };
  auto fetch = [&](int t0, BlockIn &in) {
    const int tok = min(c, T - 1 - t0);
    const __amdgpu_buffer_rsrc_t qr = rows_from(qb + t0 * q_row);
#pragma unroll
    for (int h = 0; h < kMaxGroup; ++h)
      if (h < G) in.q[h] = load16(qr, tok * (int)q_row + h * q_head + r * 16);
    in.k = load16(rows_from(kb + t0 * k_row), tok * (int)k_row + r * 16);
    in.v = load16(rows_from(vb_ + t0 * v_row), tok * (int)v_row + r * 16);
    const __amdgpu_buffer_rsrc_t gr = rows_from(gb + t0 * g_row);
#pragma unroll
    for (int j = 0; j < kGateBytes / 2; ++j) in.g[j] = load16(gr, tok * (int)g_row + r * 8 * kGateBytes + 16 * j);
  };
  auto fix_tail = [&](BlockIn &in, int t0) {
    if (t0 + kCB > T && t0 + c >= T) {
#pragma unroll
      for (int h = 0; h < kMaxGroup; ++h) in.q[h] = make_uint4(0u, 0u, 0u, 0u);
      in.k = in.v = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
      for (int j = 0; j < kGateBytes / 2; ++j) in.g[j] = make_uint4(0u, 0u, 0u, 0u);
    }
  };
  float carry[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) carry[i] = 0.f;
  auto prepare = [&](const BlockIn &in, GroupStage &st, auto second_tag) {
    constexpr bool kSecond = decltype(second_tag)::value;
    const uint4 rk = in.k, rv = in.v;
    float B[8], tot[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float x;
      if constexpr (GDT == SB_F32) x = __uint_as_float(word(in.g[i >> 2], i & 3));
      else if constexpr (GDT == SB_BF16) x = (i & 1) ? bf16_hi(word(in.g[0], i >> 1)) : bf16_lo(word(in.g[0], i >> 1));
      else x = (i & 1) ? f16_hi(word(in.g[0], i >> 1)) : f16_lo(word(in.g[0], i >> 1));
      x *= kLog2e;
      x += row_shr<1>(x);
      x += row_shr<2>(x);
      x += row_shr<4>(x);
      x += row_shr<8>(x);
      if constexpr (kSecond) x += carry[i];
      B[i] = x;
      tot[i] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane | 15) << 2, __builtin_bit_cast(int, x)));
    }
    float eq[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) eq[i] = fast_exp2(B[i]);
#pragma unroll
    for (int h = 0; h < kMaxGroup; ++h)
      if (h < G) {
        const uint4 rq = in.q[h];
        uint32_t qs[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          qs[i] = Mma<BF16>::pack(bf16_lo(word(rq, i)) * p.scale * eq[2 * i], bf16_hi(word(rq, i)) * p.scale * eq[2 * i + 1]);
        *reinterpret_cast<uint4 *>(&st.qs[h][c][8 * r]) = make_uint4(qs[0], qs[1], qs[2], qs[3]);
      }
    float kf[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      kf[2 * i] = bf16_lo(word(rk, i));
      kf[2 * i + 1] = bf16_hi(word(rk, i));
    }
    uint32_t ks[4], kl[4];
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const float x0 = kf[i] * fast_exp2(fminf(-B[i], kMaxExp * kLog2e)), x1 = kf[i + 1] * fast_exp2(fminf(-B[i + 1], kMaxExp * kLog2e));
      const uint32_t h = Mma<BF16>::pack(x0, x1);
      const uint32_t l = Mma<BF16>::pack(x0 - __uint_as_float(h << 16), x1 - __uint_as_float(h & 0xffff0000u));
      ks[i / 2] = h;
      kl[i / 2] = l;
    }
    *reinterpret_cast<uint4 *>(&st.ks[c][8 * r]) = make_uint4(ks[0], ks[1], ks[2], ks[3]);
    *reinterpret_cast<uint4 *>(&st.kl[c][8 * r]) = make_uint4(kl[0], kl[1], kl[2], kl[3]);
    *reinterpret_cast<uint4 *>(&st.vs[c][8 * r]) = rv;
    if constexpr (kSecond) {
      *reinterpret_cast<float4 *>(&st.dec[8 * r]) = make_float4(fast_exp2(tot[0]), fast_exp2(tot[1]), fast_exp2(tot[2]), fast_exp2(tot[3]));
      *reinterpret_cast<float4 *>(&st.dec[8 * r + 4]) = make_float4(fast_exp2(tot[4]), fast_exp2(tot[5]), fast_exp2(tot[6]), fast_exp2(tot[7]));
    } else {
      *reinterpret_cast<float4 *>(&st.dec[8 * r]) = make_float4(tot[0], tot[1], tot[2], tot[3]);
      *reinterpret_cast<float4 *>(&st.dec[8 * r + 4]) = make_float4(tot[4], tot[5], tot[6], tot[7]);
#pragma unroll
      for (int i = 0; i < 8; ++i) carry[i] = tot[i];
    }
  };

  auto multiply = [&](int t0, const GroupStage &st, auto second_tag) {
    constexpr bool kSecond = decltype(second_tag)::value;
    // what every head of the group shares: k-hat as the score operand, v, and the state before the block as
    // the operand of q S_0
    uint4 ka[4];
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) ka[s4] = *reinterpret_cast<const uint4 *>(&st.ks[c][32 * s4 + 8 * g]);
    uint4 vb[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const uint2 x = load_transposed(&st.vs[4 * g + (c >> 2)][32 * w + 16 * nt + 4 * (c & 3)]);
      vb[nt] = make_uint4(x.x, x.y, x.x, x.y);
    }
    uint4 sb16[4][2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const f32x4_t &a = S[2 * s4][nt], &bb = S[2 * s4 + 1][nt];
        sb16[s4][nt] = make_uint4(Mma<BF16>::pack(a[0], a[1]), Mma<BF16>::pack(a[2], a[3]),
                                  Mma<BF16>::pack(bb[0], bb[1]), Mma<BF16>::pack(bb[2], bb[3]));
      }
    // NP heads at a time, their chains of dependent matrix instructions taken in turn (a head alone is one
    // chain: four instructions for its scores, then five per output tile)
    auto heads = [&](int h0, auto np_tag) __attribute__((always_inline)) {
      constexpr int NP = decltype(np_tag)::value;
      uint4 qa[NP][4];
      f32x4_t at[NP];
#pragma unroll
      for (int u = 0; u < NP; ++u) at[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
        for (int u = 0; u < NP; ++u) {
          qa[u][s4] = *reinterpret_cast<const uint4 *>(&st.qs[h0 + u][c][32 * s4 + 8 * g]);
          at[u] = Mma<BF16>::run(ka[s4], qa[u][s4], at[u]);
        }
      uint4 pa[NP];
#pragma unroll
      for (int u = 0; u < NP; ++u) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (4 * g + i > c) at[u][i] = 0.f;
        const uint32_t h01 = Mma<BF16>::pack(at[u][0], at[u][1]), h23 = Mma<BF16>::pack(at[u][2], at[u][3]);
        pa[u] = make_uint4(h01, h23,
                           Mma<BF16>::pack(at[u][0] - __uint_as_float(h01 << 16), at[u][1] - __uint_as_float(h01 & 0xffff0000u)),
                           Mma<BF16>::pack(at[u][2] - __uint_as_float(h23 << 16), at[u][3] - __uint_as_float(h23 & 0xffff0000u)));
      }
      f32x4_t o[NP][2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int u = 0; u < NP; ++u) o[u][nt] = Mma<BF16>::run(vb[nt], pa[u], f32x4_t{0.f, 0.f, 0.f, 0.f});
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int u = 0; u < NP; ++u) o[u][nt] = Mma<BF16>::run(sb16[s4][nt], qa[u][s4], o[u][nt]);
#pragma unroll
      for (int u = 0; u < NP; ++u) {
        // (a descriptor per head: its bound drops the rows past the end of the prompt, whatever the head stride)
        const __amdgpu_buffer_rsrc_t orows = __builtin_amdgcn_make_buffer_rsrc(
            reinterpret_cast<char *>(p.out + oo) + t0 * o_row + (int64_t)(h0 + u) * o_head, 0, min(kCB, T - t0) * (int)o_row,
            0x00020000);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
          u32x2_t val;
          val.x = Mma<BF16>::pack(o[u][nt][0], o[u][nt][1]);
          val.y = Mma<BF16>::pack(o[u][nt][2], o[u][nt][3]);
          __builtin_amdgcn_raw_buffer_store_b64(val, orows, c * (int)o_row + (32 * w + 16 * nt + 4 * g) * 2, 0, 0);
        }
      }
    };
    {
      int h = 0;
      for (; h + 2 <= G; h += 2) heads(h, std::integral_constant<int, 2>{});
      if (h < G) heads(h, std::integral_constant<int, 1>{});
    }
#pragma unroll
    for (int rt = 0; rt < 8; ++rt) {
      const int tok = 4 * g + (c >> 2), dims = 32 * (rt >> 1) + 8 * (c & 3) + 4 * (rt & 1);
      const uint2 h2 = load_transposed(&st.ks[tok][dims]);
      const uint2 l2 = load_transposed(&st.kl[tok][dims]);
      const uint4 kt = make_uint4(h2.x, h2.y, l2.x, l2.y);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) S[rt][nt] = Mma<BF16>::run(kt, vb[nt], S[rt][nt]);
      if constexpr (kSecond) {
        const float4 dc = *reinterpret_cast<const float4 *>(&st.dec[32 * (rt >> 1) + 8 * g + 4 * (rt & 1)]);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          S[rt][nt][0] *= dc.x; S[rt][nt][1] *= dc.y; S[rt][nt][2] *= dc.z; S[rt][nt][3] *= dc.w;
        }
      }
    }
  };

  const int n_blocks = (T + kCB - 1) / kCB;
  const std::false_type kFirst{};
  const std::true_type kSecond{};
  BlockIn in;
  fetch(0, in);
  fix_tail(in, 0);
  prepare(in, stage[0], kFirst);
  fetch(min(1, n_blocks - 1) * kCB, in);
  int blk = 0;
  for (; blk + 1 < n_blocks; blk += 2) {
    __syncthreads();
    fix_tail(in, (blk + 1) * kCB);
    multiply(blk * kCB, stage[0], kFirst);
    prepare(in, stage[1], kSecond);
    fetch(min(blk + 2, n_blocks - 1) * kCB, in);
    __syncthreads();
    fix_tail(in, (blk + 2) * kCB);
    multiply((blk + 1) * kCB, stage[1], kSecond);
    prepare(in, stage[0], kFirst);
    fetch(min(blk + 3, n_blocks - 1) * kCB, in);
  }
  if (blk < n_blocks) {
    __syncthreads();
    multiply(blk * kCB, stage[0], kFirst);
#pragma unroll
    for (int rt = 0; rt < 8; ++rt) {
      const float4 dc = *reinterpret_cast<const float4 *>(&stage[0].dec[32 * (rt >> 1) + 8 * g + 4 * (rt & 1)]);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        S[rt][nt][0] *= fast_exp2(dc.x); S[rt][nt][1] *= fast_exp2(dc.y);
        S[rt][nt][2] *= fast_exp2(dc.z); S[rt][nt][3] *= fast_exp2(dc.w);
      }
    }
  }
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

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_hits_mu;
unsigned int *g_hits_ptr[kMaxDevices];  // per device: address of that device's copy of gla_range_hits

// Address of the current device's counter (looked up once per device), or null with the error set.
unsigned int *range_hits_ptr() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    sb_host::set_error("gla_chunk: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_hits_mu);
  if (!g_hits_ptr[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(gla_range_hits));
    if (e != hipSuccess || !ptr) {
      sb_host::set_error("gla_chunk: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    g_hits_ptr[dev] = (unsigned int *)ptr;
  }
  return g_hits_ptr[dev];
}
}  // namespace

extern "C" int sb_gla_gate_range_hits(int64_t *hits, int32_t reset) {
  using namespace sb_host;
  if (!hits) return fail(SB_ERR_INVALID, "sb_gla_gate_range_hits: null pointer");
  unsigned int *ptr = range_hits_ptr();
  if (!ptr) return SB_ERR_INVALID;
  unsigned int h = 0;
  hipError_t e = hipMemcpy(&h, ptr, sizeof(h), hipMemcpyDeviceToHost);  // waits for the work queued before it
  if (e != hipSuccess) return fail((int)e, "sb_gla_gate_range_hits: hipMemcpy: %s", hipGetErrorString(e));
  if (reset) {
    e = hipMemset(ptr, 0, sizeof(h));
    if (e != hipSuccess) return fail((int)e, "sb_gla_gate_range_hits: hipMemset: %s", hipGetErrorString(e));
  }
  *hits = (int64_t)h;
  return SB_OK;
}

namespace sb_host {

// Launch for bf16 q/k/v/out; g of any built type. Grid: one workgroup per (row, head).
// Returns SB_OK, or an error when the device's hit counter cannot be located (nothing is launched then).
int launch_gla_chunk(const sb_gla_recurrent_args *a, int64_t groups, int heads, int G, int jn, int j0, int write_state) {
  GlaChunkParams p;
  const bool check = (a->flags & SB_GLA_CHECK_GATES) != 0;
  p.range_hits = check ? range_hits_ptr() : nullptr;
  if (check && !p.range_hits) return SB_ERR_INVALID;
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
#define SB_LAUNCH(F32S, GDT)                                                                     \
  do {                                                                                           \
    if (check) hipLaunchKernelGGL((gla_chunk_kernel<F32S, GDT, true>), grid, block, 0, st, p);   \
    else hipLaunchKernelGGL((gla_chunk_kernel<F32S, GDT, false>), grid, block, 0, st, p);        \
  } while (0)
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
  return SB_OK;
}

// Shared states, one pass: grid = one workgroup per (row, state head), each forming the outputs of its G query
// heads. SB_ERR_UNSUPPORTED (nothing launched) where the group's head offsets do not fit the kernel's 32-bit
// in-block offsets; the caller then takes the launches per query head.
int launch_gla_chunk_group(const sb_gla_recurrent_args *a, int state_heads, int G) {
  if (G < 2 || G > kMaxGroup) return SB_ERR_UNSUPPORTED;
  if ((int64_t)G * a->q_stride_h * 2 >= (1LL << 30) || (int64_t)G * a->out_stride_h * 2 >= (1LL << 30) ||
      a->q_stride_h < 0 || a->out_stride_h < 0)
    return SB_ERR_UNSUPPORTED;
  GlaChunkParams p;
  p.range_hits = nullptr;
  p.q = (const uint16_t *)a->q; p.k = (const uint16_t *)a->k; p.v = (const uint16_t *)a->v; p.g = a->g;
  p.state = a->state; p.out = (uint16_t *)a->out; p.slot_idx = a->slot_idx; p.cu = a->cu_seqlens;
  p.H = state_heads; p.T = a->seq_len; p.scale = a->scale;
  p.G = G; p.jn = 1; p.j0 = 0; p.write_state = 1;
  p.q_sb = a->q_stride_b; p.q_sh = a->q_stride_h; p.q_st = a->q_stride_t;
  p.k_sb = a->k_stride_b; p.k_sh = a->k_stride_h; p.k_st = a->k_stride_t;
  p.v_sb = a->v_stride_b; p.v_sh = a->v_stride_h; p.v_st = a->v_stride_t;
  p.g_sb = a->g_stride_b; p.g_sh = a->g_stride_h; p.g_st = a->g_stride_t;
  p.o_sb = a->out_stride_b; p.o_sh = a->out_stride_h; p.o_st = a->out_stride_t;
  p.s_slot = a->state_stride_slot; p.s_head = a->state_stride_head;
  const dim3 grid((unsigned)(a->batch * (int64_t)state_heads)), block(256);
  hipStream_t st = (hipStream_t)a->stream;
  constexpr int kLds = 2 * (int)sizeof(GroupStage);
#define SB_LAUNCH(F32S, GDT)                                                                                  \
  do {                                                                                                        \
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gla_chunk_group_kernel<F32S, GDT>),    \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds);                     \
    if (e != hipSuccess) return fail((int)e, "gla_chunk_group_kernel: %s", hipGetErrorString(e));             \
    hipLaunchKernelGGL((gla_chunk_group_kernel<F32S, GDT>), grid, block, kLds, st, p);                        \
  } while (0)
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
  return SB_OK;
}

}  // namespace sb_host
