// Window-bounded single-query attention over a per-row INT8 K/V cache (codes int8
// [nb, bs, Hkv, 128], scales fp32 [nb, Hkv, bs]), split-K, matrix cores. Half the HBM bytes of
// the bf16 cache per visible key (2 x 128 B codes + 8 B scales per kv head).
//
// Same decomposition and lane layouts as the bf16 kernel (one wavefront per kv head, chunks of
// 32 keys, S^T = K Q^T then O^T += V^T P^T with P staying in-lane); what differs:
//   * codes are widened to the query's 16-bit type on the way into the matrix cores (small integers
//     are exact there); a key's K scale multiplies its score, its V scale multiplies its
//     probability, both in fp32, so nothing is rounded that the reference does not round;
//   * the contraction over head dims is order-free, so lane (g, c) takes the 32 contiguous bytes
//     [32g, 32g+32) of key c (two 16-byte loads; the query operand uses the same dim order);
//   * V codes are loaded as 8-byte row pieces (lane (g,c): its 8 keys, dims 8c..8c+7); picking byte
//     mt of each while widening IS the 8x8 transpose the bf16 kernel does with v_perm;
//   * no byte pattern of a code is a NaN, so edge chunks only clamp their TILES into the resident
//     range (rows of a resident block are always addressable) and mask by key index; scales of
//     masked keys may be stale, so masked probabilities are selected to zero, never multiplied;
//   * the append is a launch of its own (sb_kv_append_int8): the newest row has to be quantised
//     before it can be attended to;
//   * meta tokens (rows every query also attends to) are not part of the cache: they stay elements of the
//     query's type and are taken, ahead of the window, in chunks of 32 dealt round robin to the splits.
#include "common.h"
#include "mfma_util.h"
#include "swa_decode_params.h"

namespace {

using namespace sb;

constexpr float kNegInf = kNegInfF;

struct ChunkI8 {
  uint4 k[2][2];     // tile, half: bytes [32g + 16*half, +16) of key c
  uint2 v[8];        // key kk = 8g..8g+7 of the chunk: dims 8c..8c+7
  float4 ks[2], vs[2];  // scales of keys 4g..4g+3 of tile 0 / tile 1
};

// byte B of w as a float: a signed INT8 code, or an fp8 (OCP e4m3fn) code
template <int Q, int B>
__device__ __forceinline__ float code_to_float(uint32_t w) {
  if constexpr (Q == SB_KV_INT8) return (float)(int)(int8_t)(w >> (8 * B));
  else return __builtin_amdgcn_cvt_f32_fp8((int)w, B);
}

// 8 codes (two dwords) -> 8 elements of type E
template <typename E, int Q>
__device__ __forceinline__ uint4 widen8(uint32_t lo, uint32_t hi) {
  return make_uint4(Mma<E>::pack(code_to_float<Q, 0>(lo), code_to_float<Q, 1>(lo)),
                    Mma<E>::pack(code_to_float<Q, 2>(lo), code_to_float<Q, 3>(lo)),
                    Mma<E>::pack(code_to_float<Q, 0>(hi), code_to_float<Q, 1>(hi)),
                    Mma<E>::pack(code_to_float<Q, 2>(hi), code_to_float<Q, 3>(hi)));
}

__device__ __forceinline__ uint32_t word2(const uint2 &v, int i) { return i == 0 ? v.x : v.y; }

template <typename E, int Q, int B>
__device__ __forceinline__ uint4 v_column(const uint2 (&v)[8], int w) {
  return make_uint4(Mma<E>::pack(code_to_float<Q, B>(word2(v[0], w)), code_to_float<Q, B>(word2(v[1], w))),
                    Mma<E>::pack(code_to_float<Q, B>(word2(v[2], w)), code_to_float<Q, B>(word2(v[3], w))),
                    Mma<E>::pack(code_to_float<Q, B>(word2(v[4], w)), code_to_float<Q, B>(word2(v[5], w))),
                    Mma<E>::pack(code_to_float<Q, B>(word2(v[6], w)), code_to_float<Q, B>(word2(v[7], w))));
}

// 256 registers per wavefront (two per SIMD): the matrix-core results then live in ordinary registers
// and the rescale inside the loop costs no accumulator-register traffic.
// Q = SB_KV_FP8: the codes are fp8 with one scale per tensor: the K scale is folded into the softmax
// scale and the V scale into the result on the host side of the launch, nothing per key; an fp8 byte
// CAN be a NaN, so the V codes of masked keys are zeroed before they meet their zero probability.
template <typename E, int Q>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void swa_decode_split_i8_kernel(const DecodeParams p, const int G, const int Hkv) {
  const int64_t r = blockIdx.x;
  const int split = blockIdx.z;
  const int tid = threadIdx.x;
  const int kvh = blockIdx.y * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(tid >> 6);
  if (kvh >= Hkv) return;  // whole wavefront; there is no barrier in this kernel
  const int lane = tid & 63;
  const int g = lane >> 4;
  const int c = lane & 15;

  const int64_t seq = p.row_seq ? (int64_t)p.row_seq[r] : r;
  const int hi = p.seq_lens[r];
  int lo = p.window_left >= 0 ? max(0, hi - 1 - p.window_left) : 0;
  if (p.key_lo) lo = max(lo, p.key_lo[r]);
  const bool any = hi > lo;
  const int first_tile = lo >> 4;
  const int last_tile = any ? (hi - 1) >> 4 : first_tile;
  const int first_chunk = lo >> 5;
  const int n_chunks = any ? ((hi - 1) >> 5) - first_chunk + 1 : 0;
  const int cps = (n_chunks + p.n_split - 1) / p.n_split;
  const int cb = first_chunk + split * cps;
  const int ce = min(cb + cps, first_chunk + n_chunks);

  // Q^T operands: head c of the group, dims 32g + 8s .. +7 for step s; zero rows pad the group
  uint4 qb[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    qb[s] = make_uint4(0u, 0u, 0u, 0u);
    if (c < G)
      qb[s] = *reinterpret_cast<const uint4 *>(
          p.q + (r * p.q_sr + (int64_t)(kvh * G + c) * p.q_sh + 32 * g + 8 * s) * 2);
  }

  const float my_slope = (p.opt.slopes && c < G) ? p.opt.slopes[kvh * G + c] : 0.f;  // ALiBi slope of this lane's head

  f32x4_t acc[8];
#pragma unroll
  for (int mt = 0; mt < 8; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = kNegInf, l = 0.f;

  const uint32_t kv_sr32 = (uint32_t)p.kv_sr;
  const uint32_t koff = c * kv_sr32 + g * 32;
  uint32_t voff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) voff[j] = (4 * g + j) * kv_sr32 + c * 8;

  auto load_chunk = [&](int cc, ChunkI8 &ck) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int tile = min(max(2 * cc + t, first_tile), last_tile);  // resident, uniform over the wavefront
      const int i0 = tile << 4;
      const int bi = i0 / p.block_size;
      const int row = i0 - bi * p.block_size;
      const int64_t blk = p.block_table[seq * p.bt_stride + bi];
      const int64_t base = blk * p.kv_sb + (int64_t)row * p.kv_sr + (int64_t)kvh * p.kv_sh;
      const char *kp = p.k + base, *vp = p.v + base;
      ck.k[t][0] = load_stream16(kp + koff);
      ck.k[t][1] = load_stream16(kp + koff + 16);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const unsigned long long w = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long *>(vp + voff[j]));
        ck.v[4 * t + j] = make_uint2((uint32_t)w, (uint32_t)(w >> 32));
      }
      if constexpr (Q == SB_KV_INT8) {
        const int64_t sbase = (blk * Hkv + kvh) * p.block_size + row + 4 * g;
        ck.ks[t] = *reinterpret_cast<const float4 *>(p.k_scale + sbase);
        ck.vs[t] = *reinterpret_cast<const float4 *>(p.v_scale + sbase);
      }
    }
  };

  auto compute_chunk = [&](int ch, const ChunkI8 &ck) {
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint4 &a = ck.k[0][s >> 1], &b = ck.k[1][s >> 1];
      s0 = Mma<E>::run((s & 1) ? widen8<E, Q>(a.z, a.w) : widen8<E, Q>(a.x, a.y), qb[s], s0);
      s1 = Mma<E>::run((s & 1) ? widen8<E, Q>(b.z, b.w) : widen8<E, Q>(b.x, b.y), qb[s], s1);
    }
    float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
    float vsc[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
    if constexpr (Q == SB_KV_INT8) {
      const float ksc[8] = {ck.ks[0].x, ck.ks[0].y, ck.ks[0].z, ck.ks[0].w, ck.ks[1].x, ck.ks[1].y, ck.ks[1].z, ck.ks[1].w};
      const float vs8[8] = {ck.vs[0].x, ck.vs[0].y, ck.vs[0].z, ck.vs[0].w, ck.vs[1].x, ck.vs[1].y, ck.vs[1].z, ck.vs[1].w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        sc[j] *= ksc[j];
        vsc[j] = vs8[j];
      }
    }
    bool vis[8];
    const int i0 = ch << 5;
    if (p.opt.on) {  // soft cap / ALiBi (wave-uniform; the query sits at key index hi - 1)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        sc[j] = adjust_score(p.opt, sc[j], my_slope, (float)(i0 + ((j >> 2) << 4) + 4 * g + (j & 3) - (hi - 1)));
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = i0 + ((j >> 2) << 4) + 4 * g + (j & 3);
      vis[j] = i >= lo && i < hi;
      if (!vis[j]) sc[j] = kNegInf;
    }
    float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m, mx * p.scale_log2);
    const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = fast_exp2(m - m_safe);
    const bool grew = m_new > m;
    m = m_new;
    float psum = 0.f, pv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float e = fast_exp2(fmaf(sc[j], p.scale_log2, -m_safe));
      psum += e;
      pv[j] = vis[j] ? e * vsc[j] : 0.f;
    }
    uint2 vq[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) vq[j] = (Q == SB_KV_FP8 && !vis[j]) ? make_uint2(0u, 0u) : ck.v[j];
    l = fmaf(l, alpha, psum);
    if (__builtin_amdgcn_ballot_w64(grew) != 0) {
#pragma unroll
      for (int mt = 0; mt < 8; ++mt) acc[mt] *= alpha;
    }
    const uint4 pb = make_uint4(Mma<E>::pack(pv[0], pv[1]), Mma<E>::pack(pv[2], pv[3]),
                                Mma<E>::pack(pv[4], pv[5]), Mma<E>::pack(pv[6], pv[7]));
    acc[0] = Mma<E>::run(v_column<E, Q, 0>(vq, 0), pb, acc[0]);
    acc[1] = Mma<E>::run(v_column<E, Q, 1>(vq, 0), pb, acc[1]);
    acc[2] = Mma<E>::run(v_column<E, Q, 2>(vq, 0), pb, acc[2]);
    acc[3] = Mma<E>::run(v_column<E, Q, 3>(vq, 0), pb, acc[3]);
    acc[4] = Mma<E>::run(v_column<E, Q, 0>(vq, 1), pb, acc[4]);
    acc[5] = Mma<E>::run(v_column<E, Q, 1>(vq, 1), pb, acc[5]);
    acc[6] = Mma<E>::run(v_column<E, Q, 2>(vq, 1), pb, acc[6]);
    acc[7] = Mma<E>::run(v_column<E, Q, 3>(vq, 1), pb, acc[7]);
  };

  // ---- meta rows: dense element tensors [meta_len, Hkv, 128], chunk cc = rows 32cc .. 32cc+31 clamped to the
  // last row (masked by their true index). K operand in this kernel's dim order (lane (g, c): bytes
  // [64g, 64g+64) of row c), V rows as the element kernel takes them (lane (g, c): bytes [16c, 16c+16) of its
  // 8 keys, transposed in registers). The rows have no scales: meta_k_mult / meta_v_mult undo the tensor
  // scales an fp8 cache folds into scale_log2 and kv_out_scale.
  auto meta_chunk = [&](int cc) {
    const char *mk = p.meta_k + (int64_t)kvh * p.meta_sh, *mv = p.meta_v + (int64_t)kvh * p.meta_sh;
    const int last = p.meta_len - 1, i0 = cc << 5;
    const char *pk0 = mk + (int64_t)min(i0 + c, last) * p.meta_sr + g * 64;
    const char *pk1 = mk + (int64_t)min(i0 + 16 + c, last) * p.meta_sr + g * 64;
    uint4 v[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = *reinterpret_cast<const uint4 *>(mv + (int64_t)min(i0 + 4 * g + j, last) * p.meta_sr + c * 16);
      v[4 + j] = *reinterpret_cast<const uint4 *>(mv + (int64_t)min(i0 + 16 + 4 * g + j, last) * p.meta_sr + c * 16);
    }
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      s0 = Mma<E>::run(*reinterpret_cast<const uint4 *>(pk0 + s * 16), qb[s], s0);
      s1 = Mma<E>::run(*reinterpret_cast<const uint4 *>(pk1 + s * 16), qb[s], s1);
    }
    float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
    bool vis[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = i0 + ((j >> 2) << 4) + 4 * g + (j & 3);
      vis[j] = key < p.meta_len;
      float x = sc[j] * p.meta_k_mult;
      // soft cap / ALiBi: the meta rows' distance is that of the stacked second attention of the reference
      if (p.opt.on) x = adjust_score(p.opt, x, my_slope, -fabsf((float)(p.meta_bias_off + (int)r - key)));
      sc[j] = vis[j] ? x : kNegInf;
    }
    float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m, mx * p.scale_log2);
    const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = fast_exp2(m - m_safe);
    m = m_new;
    float psum = 0.f, pv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float e = fast_exp2(fmaf(sc[j], p.scale_log2, -m_safe));
      psum += e;
      pv[j] = vis[j] ? e * p.meta_v_mult : 0.f;
    }
    l = fmaf(l, alpha, psum);
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) acc[mt] *= alpha;
    const uint4 pb = make_uint4(Mma<E>::pack(pv[0], pv[1]), Mma<E>::pack(pv[2], pv[3]),
                                Mma<E>::pack(pv[4], pv[5]), Mma<E>::pack(pv[6], pv[7]));
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) acc[mt] = Mma<E>::run(v_transposed(v, mt), pb, acc[mt]);
  };
  if (p.meta_len > 0)
    for (int cc = split; cc < (p.meta_len + 31) >> 5; cc += p.n_split) meta_chunk(cc);

  // one chunk of loads in flight behind the one being computed; two register sets, the loop
  // written out for both so that neither is ever copied
  if (cb < ce) {
    ChunkI8 a, b;
    int ch = cb;
    load_chunk(ch, a);
    while (ch + 1 < ce) {
      load_chunk(ch + 1, b);
      compute_chunk(ch, a);
      load_chunk(min(ch + 2, ce - 1), a);
      compute_chunk(ch + 1, b);
      ch += 2;
    }
    if (ch < ce) compute_chunk(ch, a);
  }

  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);

  // ---- this wavefront's result: lane (g, c < G) owns head c, dims 32g + 8i + mt --------------
  if (c < G) {
    const int hq = kvh * G + c;
    if (p.n_split == 1) {
      const float inv = l > 0.f ? p.kv_out_scale / l : 0.f;
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
      const int64_t part = (r * p.Hq + hq) * p.n_split + split;
      float *dst = p.ws_acc + part * 128 + 32 * g;
      const float os = p.kv_out_scale;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        reinterpret_cast<float4 *>(dst + 8 * i)[0] = make_float4(acc[0][i] * os, acc[1][i] * os, acc[2][i] * os, acc[3][i] * os);
        reinterpret_cast<float4 *>(dst + 8 * i)[1] = make_float4(acc[4][i] * os, acc[5][i] * os, acc[6][i] * os, acc[7][i] * os);
      }
      if (g == 0) {
        p.ws_ml[part * 2] = m;
        p.ws_ml[part * 2 + 1] = l;
      }
    }
  }
}

}  // namespace

namespace sb_host {

// Launches the split kernel over an INT8 or fp8 cache (query dtype bf16 or fp16, group size <= 16, paged mode).
void launch_swa_decode_split_i8(int dtype, int kv_quant, int G, int Hkv, unsigned rows, unsigned n_split, hipStream_t st,
                                const sb::DecodeParams &p) {
  const int waves = Hkv < 4 ? Hkv : 4;
  const dim3 grid(rows, (unsigned)((Hkv + waves - 1) / waves), n_split), block(64 * waves);
  if (kv_quant == SB_KV_INT8) {
    if (dtype == SB_BF16) hipLaunchKernelGGL((swa_decode_split_i8_kernel<sb::BF16, SB_KV_INT8>), grid, block, 0, st, p, G, Hkv);
    else hipLaunchKernelGGL((swa_decode_split_i8_kernel<sb::F16, SB_KV_INT8>), grid, block, 0, st, p, G, Hkv);
  } else {
    if (dtype == SB_BF16) hipLaunchKernelGGL((swa_decode_split_i8_kernel<sb::BF16, SB_KV_FP8>), grid, block, 0, st, p, G, Hkv);
    else hipLaunchKernelGGL((swa_decode_split_i8_kernel<sb::F16, SB_KV_FP8>), grid, block, 0, st, p, G, Hkv);
  }
}

}  // namespace sb_host
