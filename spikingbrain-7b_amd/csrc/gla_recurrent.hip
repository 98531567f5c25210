// GLA recurrent step(s): S <- diag(exp g) S + k^T v ; o = (q*scale) S, state in place.
//
// One 256-thread workgroup owns the [128,128] state of one (batch row, head). A state row is
// 128 values = 32 lanes x 4 values, so the workgroup covers 8 rows per pass and 16 passes
// cover the state; each lane keeps its 16 row-quads (64 values) in registers for the whole
// call. The state therefore crosses HBM exactly twice (one read, one write) whatever T is,
// and all 16 row loads of a lane are independent, which is what hides HBM latency.
// Gate, outer product and the q.S column reduction are fused into the same pass.
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
};

__device__ __forceinline__ float load_scalar(const void *p, int64_t i, int dtype) {
  if (dtype == SB_F32) return reinterpret_cast<const float *>(p)[i];
  if (dtype == SB_BF16)
    return __uint_as_float((uint32_t) reinterpret_cast<const uint16_t *>(p)[i] << 16);
  return (float)reinterpret_cast<const _Float16 *>(p)[i];
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

template <bool kStateF32>
__global__ __launch_bounds__(256) void gla_recurrent_kernel(const GlaParams p) {
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

  float4 S[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) S[i] = load_state4<kStateF32>(sbase, (i * 8 + rg) * 32 + col4);

  for (int t = 0; t < p.T; ++t) {
    if (tid < 128) {
      s_q[tid] = load_scalar(p.q, b * p.q_sb + h * p.q_sh + t * p.q_st + tid, p.dtype) * p.scale;
      s_k[tid] = load_scalar(p.k, b * p.k_sb + h * p.k_sh + t * p.k_st + tid, p.dtype);
      s_v[tid] = load_scalar(p.v, b * p.v_sb + h * p.v_sh + t * p.v_st + tid, p.dtype);
      s_eg[tid] = expf(load_scalar(p.g, b * p.g_sb + h * p.g_sh + t * p.g_st + tid, p.g_dtype));
    }
    __syncthreads();
    const float4 vv = reinterpret_cast<const float4 *>(s_v)[col4];
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = i * 8 + rg;
      const float kk = s_k[row], eg = s_eg[row], qq = s_q[row];
      S[i].x = fmaf(eg, S[i].x, kk * vv.x);
      S[i].y = fmaf(eg, S[i].y, kk * vv.y);
      S[i].z = fmaf(eg, S[i].z, kk * vv.z);
      S[i].w = fmaf(eg, S[i].w, kk * vv.w);
      o.x = fmaf(qq, S[i].x, o.x);
      o.y = fmaf(qq, S[i].y, o.y);
      o.z = fmaf(qq, S[i].z, o.z);
      o.w = fmaf(qq, S[i].w, o.w);
    }
    reinterpret_cast<float4 *>(s_o[rg])[col4] = o;
    __syncthreads();
    if (tid < 128) {
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < 8; ++r) acc += s_o[r][tid];
      store_scalar(p.out, b * p.o_sb + h * p.o_sh + t * p.o_st + tid, p.dtype, acc);
    }
  }

#pragma unroll
  for (int i = 0; i < 16; ++i) store_state4<kStateF32>(sbase, (i * 8 + rg) * 32 + col4, S[i]);
}

}  // namespace

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

  const dim3 grid((unsigned)groups), block(256);
  if (a->state_dtype == SB_F32)
    hipLaunchKernelGGL(gla_recurrent_kernel<true>, grid, block, 0, (hipStream_t)a->stream, p);
  else
    hipLaunchKernelGGL(gla_recurrent_kernel<false>, grid, block, 0, (hipStream_t)a->stream, p);
  return check_launch("gla_recurrent_kernel");
}
