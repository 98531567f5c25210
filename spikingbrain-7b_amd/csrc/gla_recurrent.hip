// GLA recurrent step(s): S <- diag(exp g) S + k^T v ; o = (q*scale) S, state in place.
//
// One 256-thread workgroup owns the [128,128] state of one (batch row, head). A state row is
// 128 values = 32 lanes x 4 values, so the workgroup covers 8 rows per pass and 16 passes
// cover the state; each lane keeps its 16 row-quads (64 values) in registers for the whole
// call. The state therefore crosses HBM exactly twice (one read, one write) whatever T is,
// and all 16 row loads of a lane are independent, which is what hides HBM latency.
// Gate, outer product and the q.S column reduction are fused into the same pass, and in the
// call's last step each row-quad is stored as soon as it is updated.
#include <type_traits>

#include <hip/hip_ext.h>

#include "common.h"

namespace {

struct GlaParams {
  const void *q, *k, *v, *g;
  void *state;
  void *out;
  const int32_t *slot_idx;
  int H, T;
  int dtype, g_dtype;
  float scale;
  int64_t q_sb, q_sh, q_st;
  int64_t k_sb, k_sh, k_st;
  int64_t v_sb, v_sh, v_st;
  int64_t g_sb, g_sh, g_st;
  int64_t o_sb, o_sh, o_st;
  int64_t s_slot, s_head;
  const int32_t *cu;  // packed form: tokens of row b are cu[b] .. cu[b+1]-1, or null
  // Shared states: G query heads per head of k, v, g and state. H counts the heads of THIS launch: head
  // index hh of the grid stands for state head hk = hh / jn and query head hk * G + j0 + hh % jn, and the
  // final state is stored only if write_state. One state per head: G = jn = 1, j0 = 0, write_state = 1.
  int G, jn, j0, write_state;
};

// (state head, query head) of head index hh of the launch
__device__ __forceinline__ void launch_heads(const GlaParams &p, int hh, int &hk, int &h) {
  hk = hh / p.jn;
  h = hk * p.G + p.j0 + (hh - hk * p.jn);
}

// One element of a bf16 / f16 / f32 vector as float, without a branch on the type: the aligned 32-bit word
// holding the element is loaded unconditionally and the three readings of it are selected between. (With
// a branch per type the compiler cannot issue the loads of q, k, v and g together: each sits behind its
// own branch and waits out a whole memory round trip before the next is issued.)
__device__ __forceinline__ uint32_t load_scalar_raw(const void *p, int64_t i, int dtype, uint32_t &shift) {
  const char *a = reinterpret_cast<const char *>(p) + i * (dtype == SB_F32 ? 4 : 2);
  const uint32_t mis = (uint32_t)(reinterpret_cast<uintptr_t>(a) & 2u);
  shift = mis * 8u;
  return *reinterpret_cast<const uint32_t *>(a - mis);
}
__device__ __forceinline__ float scalar_value(uint32_t w, uint32_t shift, int dtype) {
  const uint32_t h = (w >> shift) & 0xffffu;
  const float f32 = __uint_as_float(w);
  const float bf = __uint_as_float(h << 16);
  const float f16 = (float)__builtin_bit_cast(_Float16, (uint16_t)h);
  return dtype == SB_F32 ? f32 : (dtype == SB_BF16 ? bf : f16);
}
__device__ __forceinline__ float load_scalar(const void *p, int64_t i, int dtype) {
  uint32_t shift;
  const uint32_t w = load_scalar_raw(p, i, dtype, shift);
  return scalar_value(w, shift, dtype);
}
__device__ __forceinline__ void store_scalar(void *p, int64_t i, int dtype, float x) {
  if (dtype == SB_F32)
    reinterpret_cast<float *>(p)[i] = x;
  else if (dtype == SB_BF16)
    reinterpret_cast<uint16_t *>(p)[i] = (uint16_t)sb::f32_to_bf16_bits(x);
  else
    reinterpret_cast<_Float16 *>(p)[i] = (_Float16)x;
}

typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

// The state is touched once per call (one read, one write): non-temporal accesses keep it from
// displacing anything useful in the caches and stream measurably faster from HBM.
template <bool kStateF32>
__device__ __forceinline__ float4 load_state4(const char *base, int idx4) {
  if (kStateF32) {
    const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(base) + idx4);
    return make_float4(v.x, v.y, v.z, v.w);
  } else {
    const u32x2_t w = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(base) + idx4);
    return make_float4(sb::bf16_lo(w.x), sb::bf16_hi(w.x), sb::bf16_lo(w.y), sb::bf16_hi(w.y));
  }
}
template <bool kStateF32>
__device__ __forceinline__ void store_state4(char *base, int idx4, float4 s) {
  if (kStateF32) {
    const f32x4_t v = {s.x, s.y, s.z, s.w};
    __builtin_nontemporal_store(v, reinterpret_cast<f32x4_t *>(base) + idx4);
  } else {
    const u32x2_t w = {sb::pack_bf16(s.x, s.y), sb::pack_bf16(s.z, s.w)};
    __builtin_nontemporal_store(w, reinterpret_cast<u32x2_t *>(base) + idx4);
  }
}

// The step that ends the call stores every row-quad of the state as soon as it is updated, so a workgroup's
// stores start while its later loads are still arriving and overlap the reduction of the outputs: on the 7B
// decode shape that alone took the update from 0.66 to 0.76 of the HBM peak (a plain streaming copy of the
// same bytes reaches 0.77-0.80 on the same GPU). Loading everything, computing, then storing everything kept
// the two directions of a workgroup apart. Occupancy: 84-96 registers, five wavefronts per SIMD; four, three or
// two (pinned through the LDS size) measured the same or slower, six (80 registers, spilling) slower.
template <bool kStateF32, bool kOneStep>
__global__ __launch_bounds__(256, kOneStep ? 4 : 3) void gla_recurrent_kernel(const GlaParams p) {
  const int b = blockIdx.x / p.H;
  const int h = blockIdx.x - b * p.H;
  const int64_t slot = p.slot_idx ? (int64_t)p.slot_idx[b] : (int64_t)b;
  if (slot < 0) return;  // no state for this row: nothing read, nothing written

  const int tid = threadIdx.x;
  const int col4 = tid & 31;  // columns 4*col4 .. 4*col4+3
  const int rg = tid >> 5;    // row within a pass

  __shared__ float s_q[128], s_k[128], s_eg[128];
  __shared__ __attribute__((aligned(16))) float s_v[128];
  __shared__ __attribute__((aligned(16))) float s_o[8][128];

  char *sbase = reinterpret_cast<char *>(p.state) +
                (slot * p.s_slot + (int64_t)h * p.s_head) * (kStateF32 ? 4 : 2);

  // q, k, v, g of a step are asked for before anything else (the first step's ahead of the state, whose 16
  // loads per lane would otherwise queue in front of them; a later step's while the step before it is
  // computed). Every thread takes part, without a branch: the lower half of the workgroup fetches q and k,
  // the upper half v and g. (Loads under `if (tid < 128)` get sunk into that branch next to their only
  // use, behind the state loads, and everything then waits for the whole state before the first store.)
  const bool lower = tid < 128;
  const int e = tid & 127;
  const void *src0 = lower ? p.q : p.v, *src1 = lower ? p.k : p.g;
  const int dt0 = p.dtype, dt1 = lower ? p.dtype : p.g_dtype;
  const int64_t off0 = (lower ? b * p.q_sb + h * p.q_sh : b * p.v_sb + h * p.v_sh) + e;
  const int64_t off1 = (lower ? b * p.k_sb + h * p.k_sh : b * p.g_sb + h * p.g_sh) + e;
  const int64_t st0 = lower ? p.q_st : p.v_st, st1 = lower ? p.k_st : p.g_st;
  float *const dst0 = (lower ? s_q : s_v) + e, *const dst1 = (lower ? s_k : s_eg) + e;
  uint32_t w0, w1, sh0, sh1;
  auto fetch = [&](const int t) {
    w0 = load_scalar_raw(src0, off0 + t * st0, dt0, sh0);
    w1 = load_scalar_raw(src1, off1 + t * st1, dt1, sh1);
  };
  fetch(0);

  float4 S[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    S[i] = load_state4<kStateF32>(sbase, (i * 8 + rg) * 32 + col4);
    __builtin_amdgcn_sched_barrier(0);  // issued in this order: the last step consumes them in this order
  }

  auto step = [&](const int t, auto last_tag) {
    constexpr bool kLast = decltype(last_tag)::value;
    {
      const float x0 = scalar_value(w0, sh0, dt0), x1 = scalar_value(w1, sh1, dt1);
      *dst0 = lower ? x0 * p.scale : x0;   // q * scale | v
      *dst1 = lower ? x1 : expf(x1);       // k | exp(g)
    }
    __syncthreads();
    if constexpr (!kLast) fetch(t + 1);
    const float4 vv = reinterpret_cast<const float4 *>(s_v)[col4];
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = i * 8 + rg;
      const float kk = s_k[row], eg = s_eg[row], qq = s_q[row];
      S[i].x = fmaf(kk, vv.x, eg * S[i].x);
      S[i].y = fmaf(kk, vv.y, eg * S[i].y);
      S[i].z = fmaf(kk, vv.z, eg * S[i].z);
      S[i].w = fmaf(kk, vv.w, eg * S[i].w);
      o.x = fmaf(qq, S[i].x, o.x);
      o.y = fmaf(qq, S[i].y, o.y);
      o.z = fmaf(qq, S[i].z, o.z);
      o.w = fmaf(qq, S[i].w, o.w);
      if constexpr (kLast) {
        store_state4<kStateF32>(sbase, row * 32 + col4, S[i]);
        // keep the quads in the order their loads were issued (loads return in order: the first quad can
        // be finished and stored while the last ones are still on their way)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    reinterpret_cast<float4 *>(s_o[rg])[col4] = o;
    __syncthreads();
    if (tid < 128) {
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < 8; ++r) acc += s_o[r][tid];
      store_scalar(p.out, b * p.o_sb + h * p.o_sh + t * p.o_st + tid, p.dtype, acc);
    }
  };
  // kOneStep: a decode step (one token) is an instantiation of its own. Its only step is reached straight
  // from the loads above, so its waits count exactly how many of them are still outstanding; behind a loop
  // over earlier steps the same code has to wait for everything in flight where the two paths meet.
  if constexpr (kOneStep) {
    step(0, std::true_type{});
  } else {
    for (int t = 0; t + 1 < p.T; ++t) step(t, std::false_type{});
    step(p.T - 1, std::true_type{});
  }
}

// ---- shared states: one state per kv head, G query heads read it -----------------------------------
// Same thread layout, update and summation order as the kernel above (a group's state and each of its
// heads' outputs come out bit-identical to what that kernel gives on repeated k, v, g), but the state
// crosses HBM once per group instead of once per query head.
constexpr int kMaxGroup = 8;

template <bool kStateF32, bool kOneStep>
__global__ __launch_bounds__(256, kOneStep ? 4 : 3) void gla_recurrent_grouped_kernel(const GlaParams p) {
  const int Hk = p.H / p.G;
  const int b = blockIdx.x / Hk;
  const int hk = blockIdx.x - b * Hk;
  const int64_t slot = p.slot_idx ? (int64_t)p.slot_idx[b] : (int64_t)b;
  if (slot < 0) return;

  const int tid = threadIdx.x;
  const int col4 = tid & 31;
  const int rg = tid >> 5;
  const int G = p.G;

  // the step's vectors in LDS: rows 0 .. G-1 = the group's q heads (scaled), then k, v, exp(g)
  __shared__ __attribute__((aligned(16))) float s_vec[kMaxGroup + 3][128];
  __shared__ __attribute__((aligned(16))) float s_o[kMaxGroup][8][128];
  float (*const s_q)[128] = s_vec;
  float *const s_k = s_vec[kMaxGroup], *const s_v = s_vec[kMaxGroup + 1], *const s_eg = s_vec[kMaxGroup + 2];

  char *sbase = reinterpret_cast<char *>(p.state) +
                (slot * p.s_slot + (int64_t)hk * p.s_head) * (kStateF32 ? 4 : 2);

  // Vectors first and one step ahead, as in the kernel above, every thread taking part without a branch:
  // the (G + 3) * 128 elements of q (G heads), k, v, g are dealt out 256 at a time; a thread whose turn
  // falls past the end fetches an element of g again and stores the same value a second time.
  constexpr int kIter = ((kMaxGroup + 3) * 128 + 255) / 256;
  const void *src[kIter];
  float *dst[kIter];
  int64_t off[kIter], stp[kIter];
  int kind[kIter];  // 0 = q (times scale), 1 = k or v (as is), 2 = gate (exp)
#pragma unroll
  for (int it = 0; it < kIter; ++it) {
    const int idx = tid + 256 * it, e = idx & 127;
    const int vi = min(idx >> 7, G + 2);
    const bool is_q = vi < G, is_k = vi == G, is_v = vi == G + 1;
    src[it] = is_q ? p.q : (is_k ? p.k : (is_v ? p.v : p.g));
    off[it] = (is_q ? b * p.q_sb + (hk * G + vi) * p.q_sh
                    : (is_k ? b * p.k_sb + hk * p.k_sh : (is_v ? b * p.v_sb + hk * p.v_sh : b * p.g_sb + hk * p.g_sh))) + e;
    stp[it] = is_q ? p.q_st : (is_k ? p.k_st : (is_v ? p.v_st : p.g_st));
    dst[it] = (is_q ? s_vec[vi] : s_vec[kMaxGroup + vi - G]) + e;
    kind[it] = is_q ? 0 : ((is_k || is_v) ? 1 : 2);
  }
  uint32_t w[kIter], sh[kIter];
  auto fetch = [&](const int t) {
#pragma unroll
    for (int it = 0; it < kIter; ++it)
      w[it] = load_scalar_raw(src[it], off[it] + t * stp[it], kind[it] == 2 ? p.g_dtype : p.dtype, sh[it]);
  };
  fetch(0);

  float4 S[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    S[i] = load_state4<kStateF32>(sbase, (i * 8 + rg) * 32 + col4);
    __builtin_amdgcn_sched_barrier(0);  // issued in this order: the last step consumes them in this order
  }

  auto step = [&](const int t, auto last_tag) {
    constexpr bool kLast = decltype(last_tag)::value;
#pragma unroll
    for (int it = 0; it < kIter; ++it) {
      const float x = scalar_value(w[it], sh[it], kind[it] == 2 ? p.g_dtype : p.dtype);
      *dst[it] = kind[it] == 0 ? x * p.scale : (kind[it] == 1 ? x : expf(x));
    }
    __syncthreads();
    if constexpr (!kLast) fetch(t + 1);
    const float4 vv = reinterpret_cast<const float4 *>(s_v)[col4];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = i * 8 + rg;
      const float kk = s_k[row], eg = s_eg[row];
      S[i].x = fmaf(kk, vv.x, eg * S[i].x);
      S[i].y = fmaf(kk, vv.y, eg * S[i].y);
      S[i].z = fmaf(kk, vv.z, eg * S[i].z);
      S[i].w = fmaf(kk, vv.w, eg * S[i].w);
      if constexpr (kLast) {  // as in the kernel above
        store_state4<kStateF32>(sbase, row * 32 + col4, S[i]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    for (int j = 0; j < G; ++j) {
      float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float qq = s_q[j][i * 8 + rg];
        o.x = fmaf(qq, S[i].x, o.x);
        o.y = fmaf(qq, S[i].y, o.y);
        o.z = fmaf(qq, S[i].z, o.z);
        o.w = fmaf(qq, S[i].w, o.w);
      }
      reinterpret_cast<float4 *>(s_o[j][rg])[col4] = o;
    }
    __syncthreads();
    for (int idx = tid; idx < G * 128; idx += 256) {
      const int j = idx >> 7, e = idx & 127;
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < 8; ++r) acc += s_o[j][r][e];
      store_scalar(p.out, b * p.o_sb + (hk * G + j) * p.o_sh + t * p.o_st + e, p.dtype, acc);
    }
  };
  // kOneStep: a decode step (one token) is an instantiation of its own. Its only step is reached straight
  // from the loads above, so its waits count exactly how many of them are still outstanding; behind a loop
  // over earlier steps the same code has to wait for everything in flight where the two paths meet.
  if constexpr (kOneStep) {
    step(0, std::true_type{});
  } else {
    for (int t = 0; t + 1 < p.T; ++t) step(t, std::false_type{});
    step(p.T - 1, std::true_type{});
  }
}

// ---- many steps per call (prompts) ---------------------------------------------------------
// The one-workgroup kernel above pays a global-memory round trip and two barriers per step. For
// prompts the state is cut into four 32-column blocks, one single-wavefront workgroup each (no
// barrier anywhere): lane = (column quad cq = lane / 8, row group rg = lane % 8) keeps rows
// 16*rg .. 16*rg+15 of columns 4*cq .. 4*cq+3 of its block (64 values), the q.S reduction over the
// row groups is three DPP adds inside each run of 8 lanes, and q, k, g, v of kSeqBlock steps are
// fetched one block ahead as 4-element vectors (13 loads per block and lane, element types fixed
// at compile time so that no load is followed by a type branch that would wait for it), then
// converted and parked in LDS for the broadcast reads. Needs 4-element alignment of every
// pointer and stride; the host falls back to the kernel above otherwise.
constexpr int kSeqBlock = 8;
constexpr int kSeqKernelMinSteps = 4;  // shorter calls (decode, speculative decode) use the kernel above

__device__ __forceinline__ float sum8(float x) {  // sum over the 8 lanes of a run; every lane gets it
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, true));
  return x;
}

// Four consecutive elements of type DT, as loaded (Raw) and as floats.
template <int DT>
struct Quad {
  using Raw = u32x2_t;
  static __device__ __forceinline__ Raw load(const void *p, int64_t i) {
    return *reinterpret_cast<const Raw *>(reinterpret_cast<const uint16_t *>(p) + i);
  }
  static __device__ __forceinline__ float4 widen(Raw w) {
    if (DT == SB_BF16) return make_float4(sb::bf16_lo(w.x), sb::bf16_hi(w.x), sb::bf16_lo(w.y), sb::bf16_hi(w.y));
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    // (through scalars: a bit cast taken directly from an element of the vector reads element 0 whichever
    // element is named)
    const unsigned int wx = w.x, wy = w.y;
    const h2 a = __builtin_bit_cast(h2, wx), b = __builtin_bit_cast(h2, wy);
    return make_float4((float)a.x, (float)a.y, (float)b.x, (float)b.y);
  }
  static __device__ __forceinline__ void store(void *p, int64_t i, float4 o) {
    Raw w;
    if (DT == SB_BF16) {
      w.x = sb::pack_bf16(o.x, o.y);
      w.y = sb::pack_bf16(o.z, o.w);
    } else {
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      const h2 a = {(_Float16)o.x, (_Float16)o.y}, b = {(_Float16)o.z, (_Float16)o.w};
      w.x = __builtin_bit_cast(unsigned int, a);
      w.y = __builtin_bit_cast(unsigned int, b);
    }
    *reinterpret_cast<Raw *>(reinterpret_cast<uint16_t *>(p) + i) = w;
  }
};
template <>
struct Quad<SB_F32> {
  using Raw = f32x4_t;
  static __device__ __forceinline__ Raw load(const void *p, int64_t i) {
    return *reinterpret_cast<const Raw *>(reinterpret_cast<const float *>(p) + i);
  }
  static __device__ __forceinline__ float4 widen(Raw w) { return make_float4(w.x, w.y, w.z, w.w); }
  static __device__ __forceinline__ void store(void *p, int64_t i, float4 o) {
    const Raw w = {o.x, o.y, o.z, o.w};
    *reinterpret_cast<Raw *>(reinterpret_cast<float *>(p) + i) = w;
  }
};

template <bool kStateF32, int DT, int GDT>
__global__ __launch_bounds__(64) void gla_sequence_kernel(const GlaParams p) {
  using In = Quad<DT>;
  using Gate = Quad<GDT>;
  const int cb = blockIdx.x & 3;
  const int bh = blockIdx.x >> 2;
  const int b = bh / p.H;
  int hk, h;
  launch_heads(p, bh - b * p.H, hk, h);
  const int64_t slot = p.slot_idx ? (int64_t)p.slot_idx[b] : (int64_t)b;
  if (slot < 0) return;
  int T = p.T;
  int64_t qo, ko, vo, go, oo;  // element offset of this (row, head)'s first token
  if (p.cu) {
    const int64_t t0 = p.cu[b];
    T = p.cu[b + 1] - (int)t0;
    qo = t0 * p.q_st; ko = t0 * p.k_st; vo = t0 * p.v_st; go = t0 * p.g_st; oo = t0 * p.o_st;
  } else {
    qo = b * p.q_sb; ko = b * p.k_sb; vo = b * p.v_sb; go = b * p.g_sb; oo = b * p.o_sb;
  }
  if (T <= 0) return;
  const int lane = threadIdx.x;
  const int rg = lane & 7, cq = lane >> 3;
  // loads: q, k, g as (step parity lane / 32, elements 4*(lane % 32) ..), v as (step lane / 8,
  // columns 4*(lane % 8) .. of this block)
  const int lstep = lane >> 5, lcol = (lane & 31) * 4;
  qo += h * p.q_sh + lcol; ko += hk * p.k_sh + lcol; go += hk * p.g_sh + lcol;
  vo += hk * p.v_sh + cb * 32 + rg * 4;
  oo += h * p.o_sh + cb * 32 + cq * 4;

  __shared__ __attribute__((aligned(16))) float s_q[kSeqBlock][128];
  __shared__ __attribute__((aligned(16))) float s_k[kSeqBlock][128];
  __shared__ __attribute__((aligned(16))) float s_e[kSeqBlock][128];
  __shared__ __attribute__((aligned(16))) float s_v[kSeqBlock][32];

  char *sbase = reinterpret_cast<char *>(p.state) +
                (slot * p.s_slot + (int64_t)hk * p.s_head) * (kStateF32 ? 4 : 2);
  float4 S[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) S[i] = load_state4<kStateF32>(sbase, (rg * 16 + i) * 32 + cb * 8 + cq);

  typename In::Raw rq[kSeqBlock / 2], rk[kSeqBlock / 2], rv;
  typename Gate::Raw rgt[kSeqBlock / 2];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < kSeqBlock / 2; ++i) {
      const int64_t t = min(t0 + 2 * i + lstep, T - 1);  // past the end: the last token again, never used
      rq[i] = In::load(p.q, qo + t * p.q_st);
      rk[i] = In::load(p.k, ko + t * p.k_st);
      rgt[i] = Gate::load(p.g, go + t * p.g_st);
    }
    rv = In::load(p.v, vo + (int64_t)min(t0 + cq, T - 1) * p.v_st);
  };
  fetch(0);
  for (int t0 = 0; t0 < T; t0 += kSeqBlock) {
#pragma unroll
    for (int i = 0; i < kSeqBlock / 2; ++i) {
      float4 x = In::widen(rq[i]);
      x.x *= p.scale; x.y *= p.scale; x.z *= p.scale; x.w *= p.scale;
      *reinterpret_cast<float4 *>(&s_q[2 * i + lstep][lcol]) = x;
      *reinterpret_cast<float4 *>(&s_k[2 * i + lstep][lcol]) = In::widen(rk[i]);
      float4 e = Gate::widen(rgt[i]);
      e.x = expf(e.x); e.y = expf(e.y); e.z = expf(e.z); e.w = expf(e.w);
      *reinterpret_cast<float4 *>(&s_e[2 * i + lstep][lcol]) = e;
    }
    *reinterpret_cast<float4 *>(&s_v[cq][rg * 4]) = In::widen(rv);
    if (t0 + kSeqBlock < T) fetch(t0 + kSeqBlock);  // in flight while this block is computed
    auto step = [&](int s) {
      const float4 vv = reinterpret_cast<const float4 *>(s_v[s])[cq];
      float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 k4 = reinterpret_cast<const float4 *>(s_k[s])[rg * 4 + j];
        const float4 e4 = reinterpret_cast<const float4 *>(s_e[s])[rg * 4 + j];
        const float4 q4 = reinterpret_cast<const float4 *>(s_q[s])[rg * 4 + j];
        const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, ee[4] = {e4.x, e4.y, e4.z, e4.w},
                    qq[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float4 &Sr = S[4 * j + r];
          Sr.x = fmaf(kk[r], vv.x, ee[r] * Sr.x);
          Sr.y = fmaf(kk[r], vv.y, ee[r] * Sr.y);
          Sr.z = fmaf(kk[r], vv.z, ee[r] * Sr.z);
          Sr.w = fmaf(kk[r], vv.w, ee[r] * Sr.w);
          o.x = fmaf(qq[r], Sr.x, o.x);
          o.y = fmaf(qq[r], Sr.y, o.y);
          o.z = fmaf(qq[r], Sr.z, o.z);
          o.w = fmaf(qq[r], Sr.w, o.w);
        }
      }
      o.x = sum8(o.x); o.y = sum8(o.y); o.z = sum8(o.z); o.w = sum8(o.w);
      if (rg == 0) In::store(p.out, oo + (int64_t)(t0 + s) * p.o_st, o);
    };
    // (the state update is written as k*v + (e*S): both operations then work in place on the
    // state's register; with e*S as the multiply-add every state register is copied once per step)
    const int steps = min(kSeqBlock, T - t0);
    for (int s = 0; s < steps; ++s) step(s);
  }
  if (!p.write_state) return;
#pragma unroll
  for (int i = 0; i < 16; ++i) store_state4<kStateF32>(sbase, (rg * 16 + i) * 32 + cb * 8 + cq, S[i]);
}

template <bool kStateF32, int DT>
void launch_sequence(const GlaParams &p, int gdt, dim3 grid, hipStream_t st) {
  if (gdt == SB_F32) gla_sequence_kernel<kStateF32, DT, SB_F32><<<grid, 64, 0, st>>>(p);
  else if (gdt == SB_BF16) gla_sequence_kernel<kStateF32, DT, SB_BF16><<<grid, 64, 0, st>>>(p);
  else gla_sequence_kernel<kStateF32, DT, SB_F16><<<grid, 64, 0, st>>>(p);
}
template <bool kStateF32>
void launch_sequence(const GlaParams &p, dim3 grid, hipStream_t st) {
  if (p.dtype == SB_F32) launch_sequence<kStateF32, SB_F32>(p, p.g_dtype, grid, st);
  else if (p.dtype == SB_BF16) launch_sequence<kStateF32, SB_BF16>(p, p.g_dtype, grid, st);
  else launch_sequence<kStateF32, SB_F16>(p, p.g_dtype, grid, st);
}

}  // namespace

namespace sb_host {
int launch_gla_chunk(const sb_gla_recurrent_args *a, int64_t groups, int heads, int G, int jn, int j0, int write_state);
int launch_gla_chunk_group(const sb_gla_recurrent_args *a, int state_heads, int G);
}

// Shared states: (row, state head) groups from which a prompt launch takes one workgroup per group.
constexpr int64_t kGroupPassMinGroups = 112;

// Calls of this many steps or more (and every packed call) with bf16 q, k, v run on the matrix cores.
constexpr int kChunkKernelMinSteps = 32;

extern "C" int sb_gla_recurrent(const sb_gla_recurrent_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_gla_recurrent: null args");
  if (a->batch < 0 || a->seq_len < 0) return fail(SB_ERR_INVALID, "sb_gla_recurrent: negative size");
  if (a->batch == 0 || a->seq_len == 0 || a->num_heads == 0) return SB_OK;
  if (!a->q || !a->k || !a->v || !a->g || !a->state || !a->out)
    return fail(SB_ERR_INVALID, "sb_gla_recurrent: null tensor pointer");
  if (a->head_dim != 128)
    return fail(SB_ERR_UNSUPPORTED, "sb_gla_recurrent: head_dim %d (only 128 is built)", a->head_dim);
  if (a->num_heads < 0) return fail(SB_ERR_INVALID, "sb_gla_recurrent: negative num_heads");
  auto known = [](int d) { return d == SB_BF16 || d == SB_F16 || d == SB_F32; };
  if (!known(a->dtype) || !known(a->g_dtype))
    return fail(SB_ERR_UNSUPPORTED, "sb_gla_recurrent: unknown dtype");
  if (a->state_dtype != SB_F32 && a->state_dtype != SB_BF16)
    return fail(SB_ERR_UNSUPPORTED, "sb_gla_recurrent: state dtype must be f32 or bf16");
  const int ssz = a->state_dtype == SB_F32 ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(a->state) & 15u) || (a->state_stride_slot * ssz) % 16 ||
      (a->state_stride_head * ssz) % 16)
    return fail(SB_ERR_INVALID, "sb_gla_recurrent: state rows must be 16-byte aligned");
  const int64_t groups = a->batch * (int64_t)a->num_heads;
  if (groups > 0x7fffffffLL) return fail(SB_ERR_UNSUPPORTED, "sb_gla_recurrent: batch*heads too large");
  const int G = a->q_heads_per_state > 1 ? a->q_heads_per_state : 1;
  if (a->q_heads_per_state < 0 || G > kMaxGroup || a->num_heads % G)
    return fail(SB_ERR_INVALID, "sb_gla_recurrent: q_heads_per_state %d must be 0..%d and divide num_heads %d",
                a->q_heads_per_state, kMaxGroup, a->num_heads);
  const int Hk = a->num_heads / G;

  GlaParams p;
  p.q = a->q; p.k = a->k; p.v = a->v; p.g = a->g;
  p.state = a->state; p.out = a->out; p.slot_idx = a->slot_idx;
  p.H = a->num_heads; p.T = a->seq_len;
  p.dtype = a->dtype; p.g_dtype = a->g_dtype; p.scale = a->scale;
  p.q_sb = a->q_stride_b; p.q_sh = a->q_stride_h; p.q_st = a->q_stride_t;
  p.k_sb = a->k_stride_b; p.k_sh = a->k_stride_h; p.k_st = a->k_stride_t;
  p.v_sb = a->v_stride_b; p.v_sh = a->v_stride_h; p.v_st = a->v_stride_t;
  p.g_sb = a->g_stride_b; p.g_sh = a->g_stride_h; p.g_st = a->g_stride_t;
  p.o_sb = a->out_stride_b; p.o_sh = a->out_stride_h; p.o_st = a->out_stride_t;
  p.s_slot = a->state_stride_slot; p.s_head = a->state_stride_head;

  p.cu = a->cu_seqlens;
  p.G = G; p.jn = 1; p.j0 = 0; p.write_state = 1;

  // the prompt kernel moves q, k, v, g, out as 4-element vectors
  auto quad_aligned = [](const void *ptr, int dt, int64_t sb_, int64_t sh, int64_t st) {
    const uintptr_t bytes = dt == SB_F32 ? 16 : 8;
    return (reinterpret_cast<uintptr_t>(ptr) % bytes) == 0 && sb_ % 4 == 0 && sh % 4 == 0 && st % 4 == 0;
  };
  const bool vectors_ok = quad_aligned(a->q, a->dtype, p.q_sb, p.q_sh, p.q_st) &&
                          quad_aligned(a->k, a->dtype, p.k_sb, p.k_sh, p.k_st) &&
                          quad_aligned(a->v, a->dtype, p.v_sb, p.v_sh, p.v_st) &&
                          quad_aligned(a->g, a->g_dtype, p.g_sb, p.g_sh, p.g_st) &&
                          quad_aligned(a->out, a->dtype, p.o_sb, p.o_sh, p.o_st);
  // the matrix-core kernel moves q, k, v, g as 16-byte pieces and out as 8-byte pieces
  auto piece_aligned = [](const void *ptr, int64_t per16, int64_t sb_, int64_t sh, int64_t st) {
    return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0 && sb_ % per16 == 0 && sh % per16 == 0 && st % per16 == 0;
  };
  const int64_t g_per16 = a->g_dtype == SB_F32 ? 4 : 8;
  const bool pieces_ok = piece_aligned(a->q, 8, p.q_sb, p.q_sh, p.q_st) && piece_aligned(a->k, 8, p.k_sb, p.k_sh, p.k_st) &&
                         piece_aligned(a->v, 8, p.v_sb, p.v_sh, p.v_st) &&
                         piece_aligned(a->g, g_per16, p.g_sb, p.g_sh, p.g_st) &&
                         piece_aligned(a->out, 8, p.o_sb, p.o_sh, p.o_st);
  if (a->dtype == SB_BF16 && pieces_ok && !(a->flags & SB_GLA_VECTOR_ONLY) &&
      (a->cu_seqlens || a->seq_len >= kChunkKernelMinSteps)) {
    // Shared states: the heads of a group each carry the recurrence for their own outputs (that keeps
    // one workgroup per query head busy), all reading the group's state. The group's first head stores
    // the final state, in a launch of its own behind the others so that no head reads a state already
    // advanced.
    int rc = SB_OK;
    // One pass per group (the state advanced once, the outputs of all its query heads formed against it) where
    // the groups alone fill the machine: one workgroup per group does 0.4 x the work of one per query head but
    // runs a single wavefront per SIMD; measured on 131 072 prompt tokens, 28 : 4 heads: 16 / 24 / 32 / 64 / 256
    // prompts 2.22 / 1.20 / 1.19 / 0.75 / 0.79 ms against 1.78 / 1.24 / 1.39 / 1.17 / 1.23; groups of 2 / 3 / 4 / 8
    // heads at 64 prompts 0.33 / 0.40 / 0.45 / 0.80 ms against 0.49 / 0.60 / 0.77 / 1.33. SB_GLA_GROUP_PASS /
    // SB_GLA_PER_HEAD choose by hand; the gate check exists only per head.
    const bool group_pass = (a->flags & SB_GLA_GROUP_PASS) ||
                            (!(a->flags & SB_GLA_PER_HEAD) && a->batch * (int64_t)Hk >= kGroupPassMinGroups);
    if (G > 1 && group_pass && !(a->flags & SB_GLA_CHECK_GATES)) {
      rc = launch_gla_chunk_group(a, Hk, G);
      if (rc == SB_OK) return check_launch("gla_chunk_group_kernel");
      if (rc != SB_ERR_UNSUPPORTED) return rc;
      rc = SB_OK;
    }
    if (G > 1) rc = launch_gla_chunk(a, a->batch * (int64_t)Hk * (G - 1), Hk * (G - 1), G, G - 1, 1, 0);
    if (G > 1 && rc == SB_OK) rc = launch_gla_chunk(a, a->batch * (int64_t)Hk, Hk, G, 1, 0, 1);
    else if (G <= 1) rc = launch_gla_chunk(a, groups, a->num_heads, 1, 1, 0, 1);
    if (rc != SB_OK) return rc;
    return check_launch("gla_chunk_kernel");
  }
  if (a->cu_seqlens && !vectors_ok)
    return fail(SB_ERR_UNSUPPORTED,
                "sb_gla_recurrent: the packed form needs pointers and strides of q, k, v, g, out aligned to 4 elements");
  if (a->cu_seqlens || (a->seq_len >= kSeqKernelMinSteps && vectors_ok)) {
    // prompts: one wavefront per (row, head, 32-column block of the state), inputs staged ahead
    if (groups * 4 > 0x7fffffffLL) return fail(SB_ERR_UNSUPPORTED, "sb_gla_recurrent: batch*heads too large");
    for (int pass = G > 1 ? 0 : 1; pass < 2; ++pass) {  // shared states: see the matrix-core launches above
      if (G > 1) {
        p.jn = pass == 0 ? G - 1 : 1;
        p.j0 = pass == 0 ? 1 : 0;
        p.write_state = pass;
        p.H = Hk * p.jn;
      }
      const dim3 sgrid((unsigned)(a->batch * p.H * 4));
      if (a->state_dtype == SB_F32)
        launch_sequence<true>(p, sgrid, (hipStream_t)a->stream);
      else
        launch_sequence<false>(p, sgrid, (hipStream_t)a->stream);
    }
    return check_launch("gla_sequence_kernel");
  }
  const hipStream_t st = (hipStream_t)a->stream;
  const bool f32s = a->state_dtype == SB_F32, one = a->seq_len == 1;
  if (G > 1) {  // decode with shared states: one workgroup per (row, state head)
    const dim3 ggrid((unsigned)(a->batch * Hk));
    if (f32s && one) hipLaunchKernelGGL((gla_recurrent_grouped_kernel<true, true>), ggrid, dim3(256), 0, st, p);
    else if (f32s) hipLaunchKernelGGL((gla_recurrent_grouped_kernel<true, false>), ggrid, dim3(256), 0, st, p);
    else if (one) hipLaunchKernelGGL((gla_recurrent_grouped_kernel<false, true>), ggrid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((gla_recurrent_grouped_kernel<false, false>), ggrid, dim3(256), 0, st, p);
    return check_launch("gla_recurrent_grouped_kernel");
  }
  const dim3 grid((unsigned)groups), block(256);
  if (one && a->profile_start_event && a->profile_stop_event) {  // timed launch: events on the kernel's own dispatch
    const hipEvent_t e0 = (hipEvent_t)a->profile_start_event, e1 = (hipEvent_t)a->profile_stop_event;
    if (f32s) hipExtLaunchKernelGGL((gla_recurrent_kernel<true, true>), grid, block, 0, st, e0, e1, 0, p);
    else hipExtLaunchKernelGGL((gla_recurrent_kernel<false, true>), grid, block, 0, st, e0, e1, 0, p);
    return check_launch("gla_recurrent_kernel");
  }
  if (f32s && one) hipLaunchKernelGGL((gla_recurrent_kernel<true, true>), grid, block, 0, st, p);
  else if (f32s) hipLaunchKernelGGL((gla_recurrent_kernel<true, false>), grid, block, 0, st, p);
  else if (one) hipLaunchKernelGGL((gla_recurrent_kernel<false, true>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((gla_recurrent_kernel<false, false>), grid, block, 0, st, p);
  return check_launch("gla_recurrent_kernel");
}
