// A caller of libsbcache's C ABI with no Python and no torch in the process: plain HIP allocations and copies,
// the structs and entry points of include/sbcache.h, and a check of the results against straightforward host
// loops in double precision. It stands for the binding a maintainer of the reference's own wrappers would write
// (the call sites it replaces are cited in include/sbcache.h). Test infrastructure: built by
// __graft_entry__.build(), run by tests/test_gpu_c_abi_host.py. Exit code 0 = every check passed.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "sbcache.h"

#define HIP_OK(call)                                                                          \
  do {                                                                                        \
    hipError_t e_ = (call);                                                                   \
    if (e_ != hipSuccess) {                                                                   \
      std::fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      std::exit(2);                                                                           \
    }                                                                                         \
  } while (0)
#define SB_CALL(call)                                                                       \
  do {                                                                                      \
    int rc_ = (call);                                                                       \
    if (rc_ != SB_OK) {                                                                     \
      std::fprintf(stderr, "%s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, rc_, sb_last_error()); \
      std::exit(3);                                                                         \
    }                                                                                       \
  } while (0)

static uint16_t to_bf16(float x) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &x, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float x;
  std::memcpy(&x, &u, 4);
  return x;
}
struct Lcg {  // uniform in [-1, 1), already rounded to bf16
  uint64_t s;
  float next() {
    s = s * 6364136223846793005ULL + 1442695040888963407ULL;
    return from_bf16(to_bf16(((s >> 40) / 8388608.0f) - 1.0f));
  }
};
template <typename T>
static T *to_device(const std::vector<T> &h) {
  T *d = nullptr;
  HIP_OK(hipMalloc(&d, h.size() * sizeof(T)));
  HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
  return d;
}
template <typename T>
static std::vector<T> to_host(const T *d, size_t n) {
  std::vector<T> h(n);
  HIP_OK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
  return h;
}
static std::vector<uint16_t> random_bf16(size_t n, Lcg &g, float scale = 1.f) {
  std::vector<uint16_t> v(n);
  for (auto &x : v) x = to_bf16(g.next() * scale);
  return v;
}

// ---- paged window attention: sb_kv_append + sb_swa_decode (two splits, so workspace and merge run too) ----
// (D = 128 with 28 : 4 heads is the 7B shape on the matrix cores; another head size or a group the vector kernel is
// not built for goes through the same entry points)
static int check_attention(const int D, const int Hq, const int Hkv) {
  const int B = 3, bs = 16, wl = 64, nb = 32, G = Hq / Hkv, width = 8;
  const int lens[B] = {40, 100, 17};  // keys of each sequence once this step's token is appended
  Lcg g{1};
  std::vector<uint16_t> kc = random_bf16((size_t)nb * bs * Hkv * D, g), vc = random_bf16((size_t)nb * bs * Hkv * D, g);
  const std::vector<uint16_t> q = random_bf16((size_t)B * Hq * D, g);
  const std::vector<uint16_t> nk = random_bf16((size_t)B * Hkv * D, g), nv = random_bf16((size_t)B * Hkv * D, g);
  std::vector<int32_t> table(B * width, 0), seq_lens(lens, lens + B);
  std::vector<int64_t> slots(B);
  for (int b = 0; b < B; ++b) {
    for (int j = 0; j * bs < lens[b]; ++j) table[b * width + j] = (7 * (b * width + j) + 3) % nb;  // a permutation
    const int i = lens[b] - 1;
    slots[b] = (int64_t)table[b * width + i / bs] * bs + i % bs;
  }
  uint16_t *d_k = to_device(kc), *d_v = to_device(vc), *d_q = to_device(q), *d_nk = to_device(nk), *d_nv = to_device(nv);
  int32_t *d_table = to_device(table), *d_lens = to_device(seq_lens);
  int64_t *d_slots = to_device(slots);
  uint16_t *d_out = nullptr;
  HIP_OK(hipMalloc(&d_out, (size_t)B * Hq * D * 2));

  sb_kv_append_args ap = {};
  ap.key = d_nk; ap.value = d_nv; ap.k_cache = d_k; ap.v_cache = d_v; ap.slot_mapping = d_slots;
  ap.num_tokens = B; ap.num_kv_heads = Hkv; ap.head_size = D; ap.block_size = bs; ap.dtype = SB_BF16;
  ap.key_stride_token = ap.value_stride_token = Hkv * D; ap.key_stride_head = ap.value_stride_head = D;
  ap.cache_stride_block = (int64_t)bs * Hkv * D; ap.cache_stride_row = Hkv * D; ap.cache_stride_head = D;
  ap.num_blocks = nb;
  SB_CALL(sb_kv_append(&ap));

  const int n_split = 2;
  const size_t ws_bytes = sb_swa_decode_workspace_bytes(B, Hq, D, n_split);
  void *d_ws = nullptr;
  HIP_OK(hipMalloc(&d_ws, ws_bytes));
  HIP_OK(hipMemset(d_ws, 0, ws_bytes));  // a workspace starts zeroed (its merge counters); calls leave it reusable
  sb_swa_decode_args a = {};
  a.q = d_q; a.k_cache = d_k; a.v_cache = d_v; a.out = d_out; a.block_table = d_table; a.seq_lens = d_lens;
  a.workspace = d_ws; a.workspace_bytes = ws_bytes;
  a.num_rows = B; a.num_q_heads = Hq; a.num_kv_heads = Hkv; a.head_size = D; a.block_size = bs;
  a.window_left = wl; a.max_seq_len = 100; a.n_split = n_split; a.dtype = SB_BF16;
  a.scale = 1.0f / std::sqrt((float)D);
  a.q_stride_row = a.out_stride_row = Hq * D; a.q_stride_head = a.out_stride_head = D;
  a.kv_stride_block = (int64_t)bs * Hkv * D; a.kv_stride_row = Hkv * D; a.kv_stride_head = D;
  a.block_table_stride = width;
  SB_CALL(sb_swa_decode(&a));
  HIP_OK(hipDeviceSynchronize());

  // host side: append, then softmax(q.K) V over the window in double
  for (int b = 0; b < B; ++b)
    for (int x = 0; x < Hkv * D; ++x) {
      kc[slots[b] * Hkv * D + x] = nk[(size_t)b * Hkv * D + x];
      vc[slots[b] * Hkv * D + x] = nv[(size_t)b * Hkv * D + x];
    }
  const std::vector<uint16_t> got_k = to_host(d_k, kc.size()), got_v = to_host(d_v, vc.size());
  if (got_k != kc || got_v != vc) {
    std::fprintf(stderr, "attention: cache contents differ after sb_kv_append\n");
    return 1;
  }
  const std::vector<uint16_t> out = to_host(d_out, (size_t)B * Hq * D);
  double worst = 0;
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < Hq; ++h) {
      const int lo = std::max(0, lens[b] - 1 - wl), kvh = h / G;
      std::vector<double> s(lens[b]);
      double mx = -1e300;
      for (int i = lo; i < lens[b]; ++i) {
        const size_t row = ((size_t)table[b * width + i / bs] * bs + i % bs) * Hkv * D + (size_t)kvh * D;
        double dot = 0;
        for (int d = 0; d < D; ++d) dot += (double)from_bf16(q[((size_t)b * Hq + h) * D + d]) * from_bf16(kc[row + d]);
        s[i] = dot * a.scale;
        mx = std::max(mx, s[i]);
      }
      double den = 0;
      std::vector<double> o(D, 0.0);
      for (int i = lo; i < lens[b]; ++i) {
        const size_t row = ((size_t)table[b * width + i / bs] * bs + i % bs) * Hkv * D + (size_t)kvh * D;
        const double p = std::exp(s[i] - mx);
        den += p;
        for (int d = 0; d < D; ++d) o[d] += p * from_bf16(vc[row + d]);
      }
      for (int d = 0; d < D; ++d)
        worst = std::max(worst, std::fabs(o[d] / den - from_bf16(out[((size_t)b * Hq + h) * D + d])));
    }
  std::printf("attention (head size %d, %d : %d heads): max abs error %.3e (bound 2e-2)\n", D, Hq, Hkv, worst);
  HIP_OK(hipFree(d_k)); HIP_OK(hipFree(d_v)); HIP_OK(hipFree(d_q)); HIP_OK(hipFree(d_nk)); HIP_OK(hipFree(d_nv));
  HIP_OK(hipFree(d_table)); HIP_OK(hipFree(d_lens)); HIP_OK(hipFree(d_slots)); HIP_OK(hipFree(d_out)); HIP_OK(hipFree(d_ws));
  return worst <= 2e-2 ? 0 : 1;
}

// ---- one GLA decode step on a slot cache: sb_gla_recurrent -------------------------------------------------
static int check_gla() {
  const int B = 3, H = 4, D = 128, slots = 5;
  const int32_t slot_of[B] = {4, -1, 1};  // the middle row has no state: skipped
  Lcg g{2};
  const std::vector<uint16_t> q = random_bf16((size_t)B * H * D, g), k = random_bf16((size_t)B * H * D, g),
                              v = random_bf16((size_t)B * H * D, g);
  std::vector<float> gate((size_t)B * H * D), state((size_t)slots * H * D * D);
  for (auto &x : gate) x = -0.05f * (1.0f + g.next());  // log-decays in (-0.1, 0]
  for (auto &x : state) x = 0.02f * g.next();
  uint16_t *d_q = to_device(q), *d_k = to_device(k), *d_v = to_device(v);
  float *d_g = to_device(gate), *d_s = to_device(state);
  int32_t *d_slot = to_device(std::vector<int32_t>(slot_of, slot_of + B));
  uint16_t *d_o = nullptr;
  HIP_OK(hipMalloc(&d_o, (size_t)B * H * D * 2));
  HIP_OK(hipMemset(d_o, 0, (size_t)B * H * D * 2));

  sb_gla_recurrent_args a = {};
  a.q = d_q; a.k = d_k; a.v = d_v; a.g = d_g; a.state = d_s; a.out = d_o; a.slot_idx = d_slot;
  a.batch = B; a.num_heads = H; a.seq_len = 1; a.head_dim = D;
  a.dtype = SB_BF16; a.g_dtype = SB_F32; a.state_dtype = SB_F32;
  a.scale = 1.0f / std::sqrt((float)D);
  a.q_stride_b = a.k_stride_b = a.v_stride_b = a.g_stride_b = a.out_stride_b = H * D;
  a.q_stride_h = a.k_stride_h = a.v_stride_h = a.g_stride_h = a.out_stride_h = D;
  a.q_stride_t = a.k_stride_t = a.v_stride_t = a.g_stride_t = a.out_stride_t = D;
  a.state_stride_slot = (int64_t)H * D * D; a.state_stride_head = (int64_t)D * D;
  a.num_slots = slots;
  SB_CALL(sb_gla_recurrent(&a));
  HIP_OK(hipDeviceSynchronize());

  const std::vector<float> got_s = to_host(d_s, state.size());
  const std::vector<uint16_t> got_o = to_host(d_o, (size_t)B * H * D);
  double worst_s = 0, worst_o = 0, s_max = 0;
  std::vector<char> touched(slots, 0);
  for (int b = 0; b < B; ++b) {
    if (slot_of[b] < 0) {
      for (int x = 0; x < H * D; ++x)
        if (got_o[(size_t)b * H * D + x] != 0) worst_o = 1e9;  // a skipped row's output is left alone
      continue;
    }
    touched[slot_of[b]] = 1;
    for (int h = 0; h < H; ++h) {
      const size_t vec = ((size_t)b * H + h) * D, mat = ((size_t)slot_of[b] * H + h) * D * D;
      std::vector<double> o(D, 0.0);
      for (int i = 0; i < D; ++i) {
        const double e = std::exp((double)gate[vec + i]), ki = from_bf16(k[vec + i]), qi = from_bf16(q[vec + i]) * (double)a.scale;
        for (int j = 0; j < D; ++j) {
          const double s_new = e * state[mat + (size_t)i * D + j] + ki * from_bf16(v[vec + j]);
          worst_s = std::max(worst_s, std::fabs(s_new - got_s[mat + (size_t)i * D + j]));
          s_max = std::max(s_max, std::fabs(s_new));
          o[j] += qi * s_new;
        }
      }
      for (int j = 0; j < D; ++j)
        worst_o = std::max(worst_o, std::fabs(o[j] - from_bf16(got_o[vec + j])) - std::fabs(o[j]) / 256.0);
    }
  }
  for (int s = 0; s < slots; ++s)
    if (!touched[s] && std::memcmp(&got_s[(size_t)s * H * D * D], &state[(size_t)s * H * D * D], (size_t)H * D * D * 4) != 0)
      worst_s = 1e9;  // slots no row points at stay bit-identical
  std::printf("gla: state max abs error %.3e (bound 1e-4 x %.3f), output error beyond bf16 rounding %.3e (bound 2e-2)\n",
              worst_s, s_max, std::max(worst_o, 0.0));
  HIP_OK(hipFree(d_q)); HIP_OK(hipFree(d_k)); HIP_OK(hipFree(d_v)); HIP_OK(hipFree(d_g)); HIP_OK(hipFree(d_s));
  HIP_OK(hipFree(d_slot)); HIP_OK(hipFree(d_o));
  return (worst_s <= 1e-4 * s_max && worst_o <= 2e-2) ? 0 : 1;
}

int main() {
  if (sb_abi_version() != SB_ABI_VERSION) {
    std::fprintf(stderr, "library ABI %d, header ABI %d\n", sb_abi_version(), SB_ABI_VERSION);
    return 4;
  }
  HIP_OK(hipSetDevice(0));
  const int bad = check_attention(128, 28, 4) + check_attention(64, 12, 4) + check_gla();
  std::printf(bad ? "FAILED\n" : "ok\n");
  return bad ? 1 : 0;
}
