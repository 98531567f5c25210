// Matrix-core helpers shared by the decode and prefill attention kernels (gfx950).
//
// v_mfma_f32_16x16x32_{bf16,f16}: D[16x16] += A[16x32] * B[32x16]; lane l holds
//   A[m = l%16][k = 8*(l/16) .. +7], B[k = 8*(l/16) .. +7][n = l%16], D[m = 4*(l/16)+i][n = l%16], i < 4.
#pragma once
#include "common.h"

namespace sb {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

template <typename E>
struct Mma;
template <>
struct Mma<BF16> {
  __device__ static __forceinline__ f32x4_t run(const uint4 &a, const uint4 &b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack(float lo, float hi) {
    bf16x2_t v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
  }
};
template <>
struct Mma<F16> {
  __device__ static __forceinline__ f32x4_t run(const uint4 &a, const uint4 &b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack(float lo, float hi) { return pack_f16(lo, hi); }
};

constexpr float kNegInfF = -__builtin_inff();

__device__ __forceinline__ uint32_t perm_lo(uint32_t hi_src, uint32_t lo_src) {
  return __builtin_amdgcn_perm(hi_src, lo_src, 0x05040100u);  // (hi_src.lo16 << 16) | lo_src.lo16
}
__device__ __forceinline__ uint32_t perm_hi(uint32_t hi_src, uint32_t lo_src) {
  return __builtin_amdgcn_perm(hi_src, lo_src, 0x07060302u);  // (hi_src.hi16 << 16) | lo_src.hi16
}
__device__ __forceinline__ uint32_t word(const uint4 &v, int i) {
  return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

// Bytes used exactly once per launch: stream them past the caches.
__device__ __forceinline__ uint4 load_stream16(const char *p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

// A operand of O^T += V^T P^T for 16-dim tile mt: an in-register transpose of this lane's 8 V rows
// (v[j] = dims 8c..8c+7 of key j) giving dim 8c+mt of the 8 keys.
__device__ __forceinline__ uint4 v_transposed(const uint4 (&v)[8], int mt) {
  const int w = mt >> 1;
  if (mt & 1)
    return make_uint4(perm_hi(word(v[1], w), word(v[0], w)), perm_hi(word(v[3], w), word(v[2], w)),
                      perm_hi(word(v[5], w), word(v[4], w)), perm_hi(word(v[7], w), word(v[6], w)));
  return make_uint4(perm_lo(word(v[1], w), word(v[0], w)), perm_lo(word(v[3], w), word(v[2], w)),
                    perm_lo(word(v[5], w), word(v[4], w)), perm_lo(word(v[7], w), word(v[6], w)));
}

}  // namespace sb
