// Shared device helpers for the gfx950 kernels of libsbcache.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sbcache.h"

namespace sb {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- bf16 / f16 bit helpers -------------------------------------------------------
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> bf16, round to nearest even (same rounding as torch's float->bfloat16).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}
__device__ __forceinline__ float f16_lo(uint32_t w) {
  return (float)__builtin_bit_cast(f16x2_t, w)[0];
}
__device__ __forceinline__ float f16_hi(uint32_t w) {
  return (float)__builtin_bit_cast(f16x2_t, w)[1];
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  f16x2_t v;
  v[0] = (_Float16)lo;
  v[1] = (_Float16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

// Element-type tags. A "pack" is 8 consecutive elements held by one lane.
struct BF16 {
  static constexpr int kBytes = 2;
  static constexpr int kPackWords = 4;  // 32-bit words per 8 elements
  __device__ static __forceinline__ float lo(uint32_t w) { return bf16_lo(w); }
  __device__ static __forceinline__ float hi(uint32_t w) { return bf16_hi(w); }
  __device__ static __forceinline__ uint32_t pack(float a, float b) { return pack_bf16(a, b); }
  __device__ static __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                           __builtin_bit_cast(bf16x2_t, b), c, false);
  }
};
struct F16 {
  static constexpr int kBytes = 2;
  static constexpr int kPackWords = 4;
  __device__ static __forceinline__ float lo(uint32_t w) { return f16_lo(w); }
  __device__ static __forceinline__ float hi(uint32_t w) { return f16_hi(w); }
  __device__ static __forceinline__ uint32_t pack(float a, float b) { return pack_f16(a, b); }
  __device__ static __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    // products and sum in fp32 (v_dot2_f32_f16 would do the same; written out so the
    // rounding is explicit)
    return fmaf(f16_hi(a), f16_hi(b), fmaf(f16_lo(a), f16_lo(b), c));
  }
};
struct F32 {
  static constexpr int kBytes = 4;
  static constexpr int kPackWords = 8;
};

// ---- DPP: all-reduce (sum) over each aligned group of 16 lanes ----------------------
template <int kCtrl>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_allreduce_sum(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror
  v += dpp_f32<0x140>(v);  // row_mirror
  return v;
}

// exp2 with the hardware instruction (inputs here are <= 0 or -inf).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The two score options flash-attn takes from the backend (vllm_hymeta/attention/meta_attention.py:665-690:
// alibi_slopes, logits_soft_cap). A raw dot product s becomes, in the units the kernels keep their scores in,
//   (cap * tanh(s * mult / cap) + slope * dist) / mult,     mult = softmax scale (times a cache's K scale),
// dist = key index - query position (<= 0 for visible keys), cap = 0: no cap. tanh(y) = 1 - 2 / (exp(2y) + 1)
// holds at both ends (exp -> inf gives 1, exp -> 0 gives -1).
struct ScoreOptions {
  float mult, inv_mult, cap, inv_cap2_log2e;  // inv_cap2_log2e = 2 log2(e) / cap
  const float *slopes;                        // [Hq] or null
  int on;                                     // 0: scores stay as they are
};
__device__ __forceinline__ float adjust_score(const ScoreOptions &o, float s, float slope, float dist) {
  float x = s * o.mult;
  if (o.cap > 0.f) {
    const float e = fast_exp2(x * o.inv_cap2_log2e);
    x = o.cap * (1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f));
  }
  return fmaf(slope, dist, x) * o.inv_mult;
}

}  // namespace sb

// Host-side error plumbing shared by the entry points.
namespace sb_host {
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);
}  // namespace sb_host
