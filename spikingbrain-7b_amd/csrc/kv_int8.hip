// Per-row symmetric INT8 for cached K/V: every (token, kv head) row of 128 values is stored as
// 128 signed bytes and one fp32 scale,
//   scale = clamp(max|x| / 127, 1e-5, 1e4),  code = clamp(round_half_even(x / scale), -128, 127),
// the arithmetic of quantize_sym (W8ASpike/window_attention.py:227-237), done once when the row
// enters the cache instead of on the whole window at every step (a row's codes depend on that
// row only, so the values attention sees are the same).
//
// One wavefront quantises the rows of one (token, K|V) for up to 4 heads: 16 lanes per head, 8
// values per lane; max|x| of a head is four xor-exchanges inside its 16 lanes.
#include "common.h"

namespace {

constexpr float kScaleMin = 1e-5f, kScaleMax = 1e4f;

template <int DT>
__device__ __forceinline__ void load8(const char *p, float (&x)[8]) {
  if constexpr (DT == SB_F32) {
    const float4 a = reinterpret_cast<const float4 *>(p)[0], b = reinterpret_cast<const float4 *>(p)[1];
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  } else {
    const uint4 w = *reinterpret_cast<const uint4 *>(p);
    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (DT == SB_BF16) {
        x[2 * i] = sb::bf16_lo(ws[i]);
        x[2 * i + 1] = sb::bf16_hi(ws[i]);
      } else {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 h = __builtin_bit_cast(h2, ws[i]);
        x[2 * i] = (float)h.x;
        x[2 * i + 1] = (float)h.y;
      }
    }
  }
}

template <int DT>
__device__ __forceinline__ void store8(char *p, const float (&x)[8]) {
  if constexpr (DT == SB_F32) {
    reinterpret_cast<float4 *>(p)[0] = make_float4(x[0], x[1], x[2], x[3]);
    reinterpret_cast<float4 *>(p)[1] = make_float4(x[4], x[5], x[6], x[7]);
  } else if constexpr (DT == SB_BF16) {
    *reinterpret_cast<uint4 *>(p) = make_uint4(sb::pack_bf16(x[0], x[1]), sb::pack_bf16(x[2], x[3]),
                                               sb::pack_bf16(x[4], x[5]), sb::pack_bf16(x[6], x[7]));
  } else {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const h2 h = {(_Float16)x[2 * i], (_Float16)x[2 * i + 1]};
      w[i] = __builtin_bit_cast(uint32_t, h);
    }
    *reinterpret_cast<uint4 *>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// scale of the 128-value row this lane's 16-lane group holds, and this lane's 8 codes (as floats)
__device__ __forceinline__ float quantise_row(const float (&x)[8], float (&code)[8]) {
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(x[i]));
#pragma unroll
  for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
  const float scale = fminf(fmaxf(amax / 127.f, kScaleMin), kScaleMax);
#pragma unroll
  for (int i = 0; i < 8; ++i) code[i] = fminf(fmaxf(rintf(x[i] / scale), -128.f), 127.f);
  return scale;
}

template <int DT>
__global__ __launch_bounds__(256) void kv_append_int8_kernel(
    const char *__restrict__ key, const char *__restrict__ value, char *__restrict__ k_cache,
    char *__restrict__ v_cache, float *__restrict__ k_scale, float *__restrict__ v_scale,
    const int64_t *__restrict__ slot_mapping, int64_t num_tokens, int num_kv_heads, int block_size,
    int64_t key_tok_b, int64_t key_head_b, int64_t val_tok_b, int64_t val_head_b, int64_t blk_b, int64_t row_b,
    int64_t head_b) {
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  const int64_t tok = wave >> 1;
  const int which = (int)(wave & 1);
  if (tok >= num_tokens) return;
  const int64_t slot = slot_mapping[tok];
  if (slot < 0) return;  // padded lane / token older than the window
  const int64_t blk = slot / block_size;
  const int off = (int)(slot - blk * block_size);
  const int h = blockIdx.y * 4 + (lane >> 4);
  const int piece = lane & 15;
  // lanes of a head beyond num_kv_heads still take part in the exchanges (on zeros)
  const bool live = h < num_kv_heads;
  constexpr int kEsz = DT == SB_F32 ? 4 : 2;
  float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, code[8];
  if (live) {
    const char *src = which ? value + tok * val_tok_b + h * val_head_b : key + tok * key_tok_b + h * key_head_b;
    load8<DT>(src + piece * 8 * kEsz, x);
  }
  const float scale = quantise_row(x, code);
  if (!live) return;
  uint32_t lo = 0, hi = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    lo |= ((uint32_t)(int)code[i] & 0xffu) << (8 * i);
    hi |= ((uint32_t)(int)code[4 + i] & 0xffu) << (8 * i);
  }
  char *dst = (which ? v_cache : k_cache) + blk * blk_b + off * row_b + h * head_b + piece * 8;
  *reinterpret_cast<uint2 *>(dst) = make_uint2(lo, hi);
  if (piece == 0) (which ? v_scale : k_scale)[(blk * num_kv_heads + h) * block_size + off] = scale;
}

// y = (code * scale) rounded to the tensor's dtype, row by row: what quantize_sym returns.
template <int DT>
__global__ __launch_bounds__(256) void quantize_sym_kernel(const char *__restrict__ in, char *__restrict__ out,
                                                           int64_t rows, int heads, int64_t in_row_b,
                                                           int64_t in_head_b, int64_t out_row_b, int64_t out_head_b) {
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  if (wave >= rows) return;
  const int h = blockIdx.y * 4 + (lane >> 4);
  const int piece = lane & 15;
  const bool live = h < heads;
  constexpr int kEsz = DT == SB_F32 ? 4 : 2;
  float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, code[8];
  if (live) load8<DT>(in + wave * in_row_b + h * in_head_b + piece * 8 * kEsz, x);
  const float scale = quantise_row(x, code);
  if (!live) return;
#pragma unroll
  for (int i = 0; i < 8; ++i) code[i] *= scale;
  store8<DT>(out + wave * out_row_b + h * out_head_b + piece * 8 * kEsz, code);
}

// ---- fp8 (OCP e4m3fn) K/V with per-tensor scales ---------------------------------------------------
// code = e4m3fn(clamp(x / scale, -448, 448)), round to nearest even: what the kv_cache_dtype="fp8"
// branch of reshape_and_cache_flash stores (vllm_hymeta/attention/meta_attention.py:790-799 with
// layer._k_scale / layer._v_scale). gfx950's v_cvt_pk_fp8_f32 is that rounding; it does not saturate,
// hence the clamp. NaN stays NaN.
__device__ __forceinline__ uint32_t to_fp8x4(float a, float b, float c, float d, float s) {
  auto q = [&](float x) { return fminf(fmaxf(x / s, -448.f), 448.f); };  // fminf/fmaxf would drop a NaN: kept below
  const float qa = a != a ? a : q(a), qb = b != b ? b : q(b), qc = c != c ? c : q(c), qd = d != d ? d : q(d);
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(qa, qb, 0, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(qc, qd, r, true);
  return (uint32_t)r;
}

template <int DT>
__global__ __launch_bounds__(256) void kv_append_fp8_kernel(
    const char *__restrict__ key, const char *__restrict__ value, char *__restrict__ k_cache,
    char *__restrict__ v_cache, const int64_t *__restrict__ slot_mapping, int64_t num_tokens, int num_kv_heads,
    int block_size, int64_t key_tok_b, int64_t key_head_b, int64_t val_tok_b, int64_t val_head_b, int64_t blk_b,
    int64_t row_b, int64_t head_b, float k_scale, float v_scale) {
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  const int64_t tok = wave >> 1;
  const int which = (int)(wave & 1);
  if (tok >= num_tokens) return;
  const int64_t slot = slot_mapping[tok];
  if (slot < 0) return;
  const int64_t blk = slot / block_size;
  const int off = (int)(slot - blk * block_size);
  const int h = blockIdx.y * 4 + (lane >> 4);
  const int piece = lane & 15;
  if (h >= num_kv_heads) return;
  constexpr int kEsz = DT == SB_F32 ? 4 : 2;
  float x[8];
  const char *src = which ? value + tok * val_tok_b + h * val_head_b : key + tok * key_tok_b + h * key_head_b;
  load8<DT>(src + piece * 8 * kEsz, x);
  const float sc = which ? v_scale : k_scale;
  char *dst = (which ? v_cache : k_cache) + blk * blk_b + off * row_b + h * head_b + piece * 8;
  *reinterpret_cast<uint2 *>(dst) = make_uint2(to_fp8x4(x[0], x[1], x[2], x[3], sc), to_fp8x4(x[4], x[5], x[6], x[7], sc));
}

// y = e4m3fn(clamp(x / scale)) * scale rounded to the tensor's dtype: what a tensor looks like after a
// round trip through the fp8 cache (or through scaled_fp8_quant, meta_attention.py:806-811, :853-869).
template <int DT>
__global__ __launch_bounds__(256) void fp8_round_kernel(const char *__restrict__ in, char *__restrict__ out,
                                                        int64_t rows, int64_t in_row_b, int64_t out_row_b, int row_vecs,
                                                        float scale) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t r = t / row_vecs;
  if (r >= rows) return;
  const int vec = (int)(t - r * row_vecs);
  constexpr int kEsz = DT == SB_F32 ? 4 : 2;
  float x[8];
  load8<DT>(in + r * in_row_b + vec * 8 * kEsz, x);
  const uint32_t lo = to_fp8x4(x[0], x[1], x[2], x[3], scale), hi = to_fp8x4(x[4], x[5], x[6], x[7], scale);
  const float y[8] = {__builtin_amdgcn_cvt_f32_fp8((int)lo, 0) * scale, __builtin_amdgcn_cvt_f32_fp8((int)lo, 1) * scale,
                      __builtin_amdgcn_cvt_f32_fp8((int)lo, 2) * scale, __builtin_amdgcn_cvt_f32_fp8((int)lo, 3) * scale,
                      __builtin_amdgcn_cvt_f32_fp8((int)hi, 0) * scale, __builtin_amdgcn_cvt_f32_fp8((int)hi, 1) * scale,
                      __builtin_amdgcn_cvt_f32_fp8((int)hi, 2) * scale, __builtin_amdgcn_cvt_f32_fp8((int)hi, 3) * scale};
  store8<DT>(out + r * out_row_b + vec * 8 * kEsz, y);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int elem_size(int dtype) {
  switch (dtype) {
    case SB_BF16:
    case SB_F16: return 2;
    case SB_F32: return 4;
    default: return 0;
  }
}

}  // namespace

extern "C" int sb_kv_append_int8(const sb_kv_append_int8_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_kv_append_int8: null args");
  if (a->num_tokens < 0) return fail(SB_ERR_INVALID, "sb_kv_append_int8: negative num_tokens");
  if (a->num_tokens == 0) return SB_OK;
  if (!a->key || !a->value || !a->k_cache || !a->v_cache || !a->k_scale || !a->v_scale || !a->slot_mapping)
    return fail(SB_ERR_INVALID, "sb_kv_append_int8: null tensor pointer");
  const int esz = elem_size(a->dtype);
  if (!esz) return fail(SB_ERR_UNSUPPORTED, "sb_kv_append_int8: unknown dtype %d", a->dtype);
  if (a->head_size != 128)
    return fail(SB_ERR_UNSUPPORTED, "sb_kv_append_int8: head_size %d (only 128 is built)", a->head_size);
  if (a->num_kv_heads <= 0 || a->block_size <= 0) return fail(SB_ERR_INVALID, "sb_kv_append_int8: non-positive shape");
  const int64_t in_strides[] = {a->key_stride_token, a->key_stride_head, a->value_stride_token, a->value_stride_head};
  for (int64_t s : in_strides)
    if ((s * esz) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_kv_append_int8: stride %lld elements is not 16-byte aligned", (long long)s);
  const int64_t c_strides[] = {a->cache_stride_block, a->cache_stride_row, a->cache_stride_head};
  for (int64_t s : c_strides)
    if (s % 8 != 0) return fail(SB_ERR_INVALID, "sb_kv_append_int8: cache stride %lld is not 8-byte aligned", (long long)s);
  if (!aligned16(a->key) || !aligned16(a->value) || !aligned16(a->k_cache) || !aligned16(a->v_cache))
    return fail(SB_ERR_INVALID, "sb_kv_append_int8: tensor base not 16-byte aligned");
  const int64_t waves = a->num_tokens * 2;
  const int64_t blocks = (waves + 3) / 4;
  if (blocks > 0x7fffffffLL) return fail(SB_ERR_UNSUPPORTED, "sb_kv_append_int8: too many tokens");
  const dim3 grid((unsigned)blocks, (unsigned)((a->num_kv_heads + 3) / 4));
#define SB_ARGS                                                                                              \
  (const char *)a->key, (const char *)a->value, (char *)a->k_cache, (char *)a->v_cache, a->k_scale, a->v_scale, \
      a->slot_mapping, a->num_tokens, a->num_kv_heads, a->block_size, a->key_stride_token *esz,              \
      a->key_stride_head *esz, a->value_stride_token *esz, a->value_stride_head *esz, a->cache_stride_block,  \
      a->cache_stride_row, a->cache_stride_head
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == SB_BF16) hipLaunchKernelGGL(kv_append_int8_kernel<SB_BF16>, grid, dim3(256), 0, st, SB_ARGS);
  else if (a->dtype == SB_F16) hipLaunchKernelGGL(kv_append_int8_kernel<SB_F16>, grid, dim3(256), 0, st, SB_ARGS);
  else hipLaunchKernelGGL(kv_append_int8_kernel<SB_F32>, grid, dim3(256), 0, st, SB_ARGS);
#undef SB_ARGS
  return check_launch("kv_append_int8_kernel");
}

extern "C" int sb_quantize_sym(const sb_quantize_sym_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_quantize_sym: null args");
  if (a->rows < 0 || a->heads < 0) return fail(SB_ERR_INVALID, "sb_quantize_sym: negative size");
  if (a->rows == 0 || a->heads == 0) return SB_OK;
  if (!a->in || !a->out) return fail(SB_ERR_INVALID, "sb_quantize_sym: null tensor pointer");
  const int esz = elem_size(a->dtype);
  if (!esz) return fail(SB_ERR_UNSUPPORTED, "sb_quantize_sym: unknown dtype %d", a->dtype);
  if (a->head_size != 128)
    return fail(SB_ERR_UNSUPPORTED, "sb_quantize_sym: head_size %d (only 128 is built)", a->head_size);
  const int64_t strides[] = {a->in_stride_row, a->in_stride_head, a->out_stride_row, a->out_stride_head};
  for (int64_t s : strides)
    if ((s * esz) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_quantize_sym: stride %lld elements is not 16-byte aligned", (long long)s);
  if (!aligned16(a->in) || !aligned16(a->out)) return fail(SB_ERR_INVALID, "sb_quantize_sym: tensor base not 16-byte aligned");
  const int64_t blocks = (a->rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return fail(SB_ERR_UNSUPPORTED, "sb_quantize_sym: too many rows");
  const dim3 grid((unsigned)blocks, (unsigned)((a->heads + 3) / 4));
#define SB_ARGS                                                                                         \
  (const char *)a->in, (char *)a->out, a->rows, a->heads, a->in_stride_row *esz, a->in_stride_head *esz, \
      a->out_stride_row *esz, a->out_stride_head *esz
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == SB_BF16) hipLaunchKernelGGL(quantize_sym_kernel<SB_BF16>, grid, dim3(256), 0, st, SB_ARGS);
  else if (a->dtype == SB_F16) hipLaunchKernelGGL(quantize_sym_kernel<SB_F16>, grid, dim3(256), 0, st, SB_ARGS);
  else hipLaunchKernelGGL(quantize_sym_kernel<SB_F32>, grid, dim3(256), 0, st, SB_ARGS);
#undef SB_ARGS
  return check_launch("quantize_sym_kernel");
}

extern "C" int sb_kv_append_fp8(const sb_kv_append_fp8_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_kv_append_fp8: null args");
  if (a->num_tokens < 0) return fail(SB_ERR_INVALID, "sb_kv_append_fp8: negative num_tokens");
  if (a->num_tokens == 0) return SB_OK;
  if (!a->key || !a->value || !a->k_cache || !a->v_cache || !a->slot_mapping)
    return fail(SB_ERR_INVALID, "sb_kv_append_fp8: null tensor pointer");
  const int esz = elem_size(a->dtype);
  if (!esz) return fail(SB_ERR_UNSUPPORTED, "sb_kv_append_fp8: unknown dtype %d", a->dtype);
  if (a->head_size != 128)
    return fail(SB_ERR_UNSUPPORTED, "sb_kv_append_fp8: head_size %d (only 128 is built)", a->head_size);
  if (a->num_kv_heads <= 0 || a->block_size <= 0) return fail(SB_ERR_INVALID, "sb_kv_append_fp8: non-positive shape");
  if (!(a->k_scale > 0.f) || !(a->v_scale > 0.f)) return fail(SB_ERR_INVALID, "sb_kv_append_fp8: scales must be positive");
  const int64_t in_strides[] = {a->key_stride_token, a->key_stride_head, a->value_stride_token, a->value_stride_head};
  for (int64_t s : in_strides)
    if ((s * esz) % 16 != 0)
      return fail(SB_ERR_INVALID, "sb_kv_append_fp8: stride %lld elements is not 16-byte aligned", (long long)s);
  const int64_t c_strides[] = {a->cache_stride_block, a->cache_stride_row, a->cache_stride_head};
  for (int64_t s : c_strides)
    if (s % 8 != 0) return fail(SB_ERR_INVALID, "sb_kv_append_fp8: cache stride %lld is not 8-byte aligned", (long long)s);
  if (!aligned16(a->key) || !aligned16(a->value) || !aligned16(a->k_cache) || !aligned16(a->v_cache))
    return fail(SB_ERR_INVALID, "sb_kv_append_fp8: tensor base not 16-byte aligned");
  const int64_t blocks = (a->num_tokens * 2 + 3) / 4;
  if (blocks > 0x7fffffffLL) return fail(SB_ERR_UNSUPPORTED, "sb_kv_append_fp8: too many tokens");
  const dim3 grid((unsigned)blocks, (unsigned)((a->num_kv_heads + 3) / 4));
#define SB_ARGS                                                                                                \
  (const char *)a->key, (const char *)a->value, (char *)a->k_cache, (char *)a->v_cache, a->slot_mapping,         \
      a->num_tokens, a->num_kv_heads, a->block_size, a->key_stride_token *esz, a->key_stride_head *esz,          \
      a->value_stride_token *esz, a->value_stride_head *esz, a->cache_stride_block, a->cache_stride_row,         \
      a->cache_stride_head, a->k_scale, a->v_scale
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == SB_BF16) hipLaunchKernelGGL(kv_append_fp8_kernel<SB_BF16>, grid, dim3(256), 0, st, SB_ARGS);
  else if (a->dtype == SB_F16) hipLaunchKernelGGL(kv_append_fp8_kernel<SB_F16>, grid, dim3(256), 0, st, SB_ARGS);
  else hipLaunchKernelGGL(kv_append_fp8_kernel<SB_F32>, grid, dim3(256), 0, st, SB_ARGS);
#undef SB_ARGS
  return check_launch("kv_append_fp8_kernel");
}

extern "C" int sb_fp8_round(const void *in, void *out, int64_t rows, int64_t row_elems, int64_t in_stride_row,
                            int64_t out_stride_row, int32_t dtype, float scale, void *stream) {
  using namespace sb_host;
  if (rows < 0 || row_elems < 0) return fail(SB_ERR_INVALID, "sb_fp8_round: negative size");
  if (rows == 0 || row_elems == 0) return SB_OK;
  if (!in || !out) return fail(SB_ERR_INVALID, "sb_fp8_round: null tensor pointer");
  const int esz = elem_size(dtype);
  if (!esz) return fail(SB_ERR_UNSUPPORTED, "sb_fp8_round: unknown dtype %d", dtype);
  if (row_elems % 8 != 0 || (in_stride_row * esz) % 16 != 0 || (out_stride_row * esz) % 16 != 0 || !aligned16(in) ||
      !aligned16(out))
    return fail(SB_ERR_INVALID, "sb_fp8_round: rows must be whole 8-element vectors at 16-byte aligned addresses");
  if (!(scale > 0.f)) return fail(SB_ERR_INVALID, "sb_fp8_round: scale must be positive");
  const int row_vecs = (int)(row_elems / 8);
  const int64_t blocks = (rows * row_vecs + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(SB_ERR_UNSUPPORTED, "sb_fp8_round: too many rows");
  const dim3 grid((unsigned)blocks);
  hipStream_t st = (hipStream_t)stream;
#define SB_ARGS (const char *)in, (char *)out, rows, in_stride_row *esz, out_stride_row *esz, row_vecs, scale
  if (dtype == SB_BF16) hipLaunchKernelGGL(fp8_round_kernel<SB_BF16>, grid, dim3(256), 0, st, SB_ARGS);
  else if (dtype == SB_F16) hipLaunchKernelGGL(fp8_round_kernel<SB_F16>, grid, dim3(256), 0, st, SB_ARGS);
  else hipLaunchKernelGGL(fp8_round_kernel<SB_F32>, grid, dim3(256), 0, st, SB_ARGS);
#undef SB_ARGS
  return check_launch("fp8_round_kernel");
}
