// Device-side decode-step advance for the sliding-window paged cache.
//
// The window-aware analogue of ops.advance_step_flashattn as called from
// vllm_hymeta/attention/meta_attention.py:338-409: every sequence of the batch takes one more token, and
// the step's seq_lens, slot_mapping and block tables are produced on the GPU, so that consecutive decode
// steps (and a captured graph of them) need no host-side metadata rebuild. Unlike the reference's kernel,
// which only bumps lengths and looks slots up in pre-grown tables, this one also does the window
// bookkeeping of the block manager: it evicts the blocks that left the window and allocates the block a
// sequence grows into, with exactly the host manager's policy - sequences in batch-row order, each one
// first pushing its evicted block ids (lowest logical block first) on the LIFO free stack, then popping
// the id for its new block - so device-advanced and host-advanced state stay bit-identical.
//
// Kernel 1 (one workgroup): per row, in parallel, what has to be evicted / allocated; then ONE thread
// replays the stack operations in row order against an LDS copy of the stack's top (a push followed by a
// pop never touches global memory); then, in parallel, the new lengths and slots.
// Kernel 2 (one workgroup per row): the window-ordered block table rows.
#include "common.h"

namespace {

struct AdvanceParams {
  int64_t *n_tokens;     // [B] tokens seen so far (in/out)
  int32_t *lo, *hi;      // [B] lowest / highest resident logical block, hi < lo = none (in/out)
  int32_t *ring;         // [B, R] physical id of logical block j at ring[b][j % R] (in/out)
  int32_t *free_stack;   // [num_blocks] free ids, next allocation = free_stack[top - 1] (in/out)
  int32_t *free_top;     // [1] (in/out)
  int64_t *slot_mapping; // [B] out
  int32_t *seq_lens;     // [B] out: keys visible through the table, newest token included
  int32_t *block_tables; // [B, table_width] out
  int32_t *status;       // [1] out, sticky: 1 = out of blocks, 2 = ring overflow
  int B, R, block_size, window_left, table_width, num_blocks;
};

constexpr int kRowsPerPass = 1024;  // rows handled per pass of the single workgroup
constexpr int kTopCache = 4096;     // stack entries simulated in LDS

__global__ __launch_bounds__(1024) void window_advance_kernel(const AdvanceParams p) {
  __shared__ int s_evict_n[kRowsPerPass];    // blocks the row evicts
  __shared__ int s_evict_lo[kRowsPerPass];   // first logical block it evicts
  __shared__ int s_evict_id[kRowsPerPass];   // physical id of the first of them (fetched in parallel)
  __shared__ int s_alloc[kRowsPerPass];      // logical block it allocates, -1 = none
  __shared__ int s_newid[kRowsPerPass];      // physical id that block got
  __shared__ int s_cache[kTopCache];         // stack entries [cache_base, cache_base + cache_n)
  __shared__ int s_work[kRowsPerPass];       // rows of this pass that evict or allocate, in row order
  __shared__ int s_wave_work[kRowsPerPass / 64];
  __shared__ int s_top, s_cache_base, s_cache_n, s_status;

  const int tid = threadIdx.x;
  const int bs = p.block_size, wl = p.window_left, R = p.R;
  if (tid == 0) {
    s_top = *p.free_top;
    s_cache_base = s_top;
    s_cache_n = 0;
    s_status = 0;
  }
  __syncthreads();

  for (int r0 = 0; r0 < p.B; r0 += kRowsPerPass) {
    const int r = r0 + tid;
    int64_t p0 = 0;
    int lo = 0, hi = -1;
    bool has_work = false;
    // ---- per row: eviction range and allocation need (block_manager policy) ------------------
    if (r < p.B) {
      p0 = p.n_tokens[r];
      lo = p.lo[r];
      hi = p.hi[r];
      const int64_t lo_new64 = (p0 - wl) / bs;
      const int lo_new = p0 - wl > 0 ? (int)lo_new64 : 0;
      const int ev_end = min(lo_new, hi + 1);
      const int lo_old = lo;
      s_evict_lo[tid] = lo;
      s_evict_n[tid] = max(0, ev_end - lo);
      if (ev_end > lo) s_evict_id[tid] = p.ring[(int64_t)r * R + lo % R];
      if (hi >= lo) {
        lo = max(lo, lo_new);
        if (lo > hi) { lo = 0; hi = -1; }
      }
      const int jb = (int)(p0 / bs);
      if (hi < lo) { lo = jb; hi = jb - 1; }
      if (jb > hi) {
        s_alloc[tid] = jb;
        if (jb - lo + 1 > R) atomicOr(&s_status, 2);
        hi = jb;
      } else {
        s_alloc[tid] = -1;
      }
      has_work = ev_end > lo_old || s_alloc[tid] >= 0;
    }
    // Most rows of a decode step neither evict nor allocate (one in block_size does): list the ones that
    // do, still in row order, so that the serial replay below walks only those.
    const unsigned long long work_mask = __ballot(has_work);
    if ((tid & 63) == 0) s_wave_work[tid >> 6] = __popcll(work_mask);
    __syncthreads();
    int n_work = 0;
    {
      int before = 0;
      for (int w = 0; w < kRowsPerPass / 64; ++w) {
        const int c = s_wave_work[w];
        before += w < (tid >> 6) ? c : 0;
        n_work += c;
      }
      if (has_work) s_work[before + __popcll(work_mask & ((1ull << (tid & 63)) - 1))] = tid;
    }
    __syncthreads();
    // ---- one thread replays pushes and pops in row order ---------------------------------------
    if (tid == 0) {
      int top = s_top, base = s_cache_base, n = s_cache_n;
      for (int w = 0; w < n_work; ++w) {
        const int i = s_work[w];
        const int en = s_evict_n[i];
        for (int k = 0; k < en; ++k) {
          const int id = k == 0 ? s_evict_id[i] : p.ring[(int64_t)(r0 + i) * R + (s_evict_lo[i] + k) % R];
          if (n == kTopCache) {  // cache full: spill it to the global stack and start afresh
            for (int u = 0; u < n; ++u) p.free_stack[base + u] = s_cache[u];
            base += n;
            n = 0;
          }
          s_cache[n++] = id;
          ++top;
        }
        const int jb = s_alloc[i];
        if (jb >= 0) {
          if (top == 0) {
            // No free block: the row does not take its token (see below); its ring entry is left as it is,
            // so no block another sequence owns is handed out or written to.
            s_status |= 1;
            s_newid[i] = -1;
          } else {
            int id;
            --top;
            if (n > 0) {
              id = s_cache[--n];
            } else {
              id = p.free_stack[top];
              base = top;
            }
            p.ring[(int64_t)(r0 + i) * R + jb % R] = id;
            s_newid[i] = id;
          }
        }
      }
      s_top = top;
      s_cache_base = base;
      s_cache_n = n;
    }
    __threadfence_block();
    __syncthreads();
    // ---- per row: new state, slot and visible length -----------------------------------------
    if (r < p.B) {
      const int jb = (int)(p0 / bs);
      // (the freshly allocated id comes from LDS: the global ring entry was written by another lane)
      const int id = s_alloc[tid] >= 0 ? s_newid[tid] : p.ring[(int64_t)r * R + jb % R];
      if (id < 0) {
        // Out of blocks (status bit 0 is set): the row's token is not taken. Its slot is the pad slot, so
        // the step's append skips it; its length counts the cached keys only; its token count does not move
        // (the next advance tries again); what left the window stays evicted. The row's attention output
        // of this step is meaningless and the caller finds out from the status word.
        hi = jb - 1;
        p.slot_mapping[r] = -1;
        p.seq_lens[r] = (int)max((int64_t)0, p0 - (int64_t)lo * bs);
        p.lo[r] = lo;
        p.hi[r] = hi;
      } else {
        p.slot_mapping[r] = (int64_t)id * bs + (p0 - (int64_t)jb * bs);
        p.seq_lens[r] = (int)(p0 + 1 - (int64_t)lo * bs);
        p.n_tokens[r] = p0 + 1;
        p.lo[r] = lo;
        p.hi[r] = hi;
      }
    }
    __syncthreads();
  }
  if (tid == 0) {
    for (int u = 0; u < s_cache_n; ++u) p.free_stack[s_cache_base + u] = s_cache[u];
    *p.free_top = s_top;
    if (s_status) atomicOr(p.status, s_status);
  }
}

// block_tables[b][j] = physical id of the j-th resident block (oldest first), 0 beyond the last
__global__ __launch_bounds__(256) void window_tables_kernel(const AdvanceParams p) {
  const int b = blockIdx.x;
  const int lo = p.lo[b], hi = p.hi[b];
  const int32_t *ring = p.ring + (int64_t)b * p.R;
  int32_t *row = p.block_tables + (int64_t)b * p.table_width;
  for (int j = threadIdx.x; j < p.table_width; j += blockDim.x)
    row[j] = (lo + j <= hi) ? ring[(lo + j) % p.R] : 0;
}

}  // namespace

extern "C" int sb_window_advance(const sb_window_advance_args *a) {
  using namespace sb_host;
  if (!a) return fail(SB_ERR_INVALID, "sb_window_advance: null args");
  if (a->batch < 0) return fail(SB_ERR_INVALID, "sb_window_advance: negative batch");
  if (a->batch == 0) return SB_OK;
  if (!a->n_tokens || !a->lo || !a->hi || !a->ring || !a->free_stack || !a->free_top || !a->slot_mapping ||
      !a->seq_lens || !a->block_tables || !a->status)
    return fail(SB_ERR_INVALID, "sb_window_advance: null pointer");
  if (a->block_size < 16 || a->block_size % 16 != 0)
    return fail(SB_ERR_INVALID, "sb_window_advance: block_size %d must be a multiple of 16", a->block_size);
  if (a->window_left < 0) return fail(SB_ERR_INVALID, "sb_window_advance: window_left must be >= 0");
  if (a->ring_blocks < a->window_left / a->block_size + 2)
    return fail(SB_ERR_INVALID, "sb_window_advance: ring of %d blocks cannot hold a window of %d tokens",
                a->ring_blocks, a->window_left);
  if (a->table_width <= 0 || a->num_blocks <= 0 || a->batch > 0x7fffffffLL)
    return fail(SB_ERR_INVALID, "sb_window_advance: bad table_width / num_blocks / batch");

  AdvanceParams p;
  p.n_tokens = a->n_tokens; p.lo = a->lo; p.hi = a->hi; p.ring = a->ring;
  p.free_stack = a->free_stack; p.free_top = a->free_top;
  p.slot_mapping = a->slot_mapping; p.seq_lens = a->seq_lens; p.block_tables = a->block_tables;
  p.status = a->status;
  p.B = (int)a->batch; p.R = a->ring_blocks; p.block_size = a->block_size; p.window_left = a->window_left;
  p.table_width = a->table_width; p.num_blocks = a->num_blocks;
  hipStream_t st = (hipStream_t)a->stream;
  hipLaunchKernelGGL(window_advance_kernel, dim3(1), dim3(1024), 0, st, p);
  int rc = check_launch("window_advance_kernel");
  if (rc != SB_OK) return rc;
  hipLaunchKernelGGL(window_tables_kernel, dim3((unsigned)p.B), dim3(256), 0, st, p);
  return check_launch("window_tables_kernel");
}
