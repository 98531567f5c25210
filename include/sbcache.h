/*
 * sbcache.h — C ABI of libsbcache.so: the decode-time cache hot path of a
 * SpikingBrain-7B-shaped hybrid model (sliding-window paged KV cache, window-bounded
 * paged decode attention, GLA recurrent-state update) as hand-written HIP kernels for
 * gfx950 (MI355X).
 *
 * Conventions
 *   - every pointer named in an args struct is a DEVICE pointer unless stated otherwise;
 *   - strides are in ELEMENTS of the tensor's dtype, sizes are element counts;
 *   - no entry point allocates, frees or synchronises; kernels are enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL = the null stream);
 *   - return value: 0 = launched; negative = rejected before launch (SB_ERR_*);
 *     positive = the hipError_t reported by the launch. sb_last_error() gives the text
 *     of the most recent failure on the calling thread;
 *   - no global mutable state: entry points are re-entrant.
 *
 * Each entry point cites the reference interface it replaces (paths relative to the
 * BICLab/SpikingBrain-7B tree).
 */
#ifndef SBCACHE_H
#define SBCACHE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SB_ABI_VERSION 3

enum sb_dtype { SB_BF16 = 0, SB_F16 = 1, SB_F32 = 2 };

enum sb_status {
  SB_OK = 0,
  SB_ERR_INVALID = -1,     /* malformed argument (null pointer, bad size, misalignment) */
  SB_ERR_UNSUPPORTED = -2, /* a shape / dtype the kernels are not instantiated for */
  SB_ERR_WORKSPACE = -3    /* caller workspace too small */
};

/* ABI version of the loaded library (== SB_ABI_VERSION of the header it was built from). */
int sb_abi_version(void);

/* Text of the last failure on this thread ("" if none). Host pointer, valid until the next call. */
const char *sb_last_error(void);

/* ------------------------------------------------------------------------------------
 * KV append — scatter new key/value rows into the paged cache at slot_mapping.
 * Replaces torch.ops._C_cache_ops.reshape_and_cache_flash as called from
 * vllm_hymeta/attention/meta_attention.py:790-799.
 *   key/value     [num_tokens, num_kv_heads, head_size]   (token and head strides given)
 *   k_cache/v_cache [num_blocks, block_size, num_kv_heads, head_size] (strides given;
 *                 the two halves of the (2, nb, bs, Hkv, D) tensor of meta_attention.py:92)
 *   slot_mapping  [num_tokens] int64; slot = block*block_size + offset; slot < 0 skips the
 *                 token (PAD_SLOT_ID, meta_attention.py:558).
 * Pure byte copy: bit-exact. head_size*sizeof(dtype) must be a multiple of 16 and all
 * row starts 16-byte aligned.
 * ------------------------------------------------------------------------------------ */
typedef struct sb_kv_append_args {
  const void *key;
  const void *value;
  void *k_cache;
  void *v_cache;
  const int64_t *slot_mapping;
  int64_t num_tokens;
  int32_t num_kv_heads;
  int32_t head_size;
  int32_t block_size;
  int32_t dtype; /* enum sb_dtype */
  int64_t key_stride_token, key_stride_head;
  int64_t value_stride_token, value_stride_head;
  int64_t cache_stride_block, cache_stride_row, cache_stride_head;
  int64_t num_blocks; /* bound for host-side validation only */
  void *stream;
} sb_kv_append_args;

int sb_kv_append(const sb_kv_append_args *args);

/* ------------------------------------------------------------------------------------
 * Window-bounded single-query attention over the paged (or a dense) KV cache.
 * Replaces flash_attn_2_cuda.fwd_kvcache as called from
 * vllm_hymeta/attention/fa_kernel_metatoken.py:84-105 (via :157-168 and
 * meta_attention.py:965-981), with causal=True and window_size=(window_left, -1); and the
 * decode step of hf_7B_model/window_attention_sdpa.py:186-214 on a dense cache.
 *
 * One "query row" r = one query token. Its keys are indices i in [0, seq_lens[r]) of
 * sequence row_seq[r]; the query sits at index seq_lens[r]-1; key i is visible iff
 *     max(seq_lens[r]-1-window_left, key_lo[r]) <= i <= seq_lens[r]-1
 * (window_left < 0 = unbounded; key_lo NULL = 0). A row with no visible key yields zeros
 * (and lse = -inf), which is what nan_to_num gives at window_attention_sdpa.py:213-214.
 *
 * Key addressing, element offset of key i / kv-head h of sequence s:
 *   paged  (block_table != NULL): blk = block_table[s*block_table_stride + i/block_size]
 *          blk*kv_stride_block + (i%block_size)*kv_stride_row + h*kv_stride_head
 *   dense  (block_table == NULL): (kv_start[s] + i)*kv_stride_row + h*kv_stride_head
 * block_size must be a multiple of 16 in paged mode (meta_attention.py:88-91).
 *
 * out[r, hq, :] = softmax_i(scale * q[r,hq,:]·K[i,hq/G,:]) · V[i,hq/G,:], fp32 accumulate,
 * rounded once to dtype. lse (optional, fp32 [num_rows, num_q_heads], natural log) is the
 * log-sum-exp of the scaled scores, the quantity fa_kernel_metatoken.py:110-122 merges on.
 *
 * The kernel splits each row's window into n_split parts and merges them; partials live
 * in `workspace` (sb_swa_decode_workspace_bytes). n_split = 0 picks a split count from
 * the shapes alone (never from device data), so the call is graph-capturable.
 * The first 64 KiB of the workspace are reserved for SB_DECODE_MERGE_IN_KERNEL (arrival counters):
 * with that flag they must be ZERO when a workspace is used for the first time (hipMemset it once
 * after allocating it); every call leaves them zero again, whatever its shape, so a workspace can be
 * reused by any later call on the stream. (Their last word is a sticky fault flag: non-zero means
 * partial results were merged across XCDs, which the launch geometry rules out; tests assert it
 * stays zero.) Without the flag the region is not touched.
 * head_size: 32 to 256 in steps of 32, the list of vllm_hymeta/attention/meta_attention.py:57-59. At 128
 * bf16/fp16 run on the matrix cores with any GQA group size num_q_heads/num_kv_heads <= 16; fp32,
 * SB_DECODE_FORCE_VALU, larger groups and every other head size run on the vector ALUs (8, 16 or 32
 * lanes per key row; built for 1, 2, 4, 7 or 8 query heads per workgroup, any other group size is cut
 * into parts of one of these). Byte-code caches (kv_quant) are built for 128 and groups <= 16 only.
 * ------------------------------------------------------------------------------------ */
#define SB_KV_NONE 0
#define SB_KV_INT8 1
#define SB_KV_FP8 2
#define SB_DECODE_FORCE_VALU 1 /* bf16/fp16: use the vector-ALU split kernel instead of the matrix-core one */
/* bf16/fp16, n_split > 1, up to 1024 rows: cut the chunks of ALL rows, laid end to end, into equal runs
 * (one per CU) instead of cutting every row into n_split runs, so that neither rows of different lengths
 * nor a row count that fits the CUs badly (96 rows x 3 splits = 256 + 32 workgroups) leave CUs idle:
 * up to 2x faster on ragged batches, 20-30 % on even batches of such sizes, about 5 % slower where
 * rows x splits fills the CUs exactly (see sb_swa_decode_prefer_balanced). Same results up to fp32
 * summation order; same workspace size. Pass n_split = 2 when the fixed split would not split at all
 * (the balanced split always goes through partial results and the merge). */
#define SB_DECODE_BALANCED 2
/* bf16/fp16 fixed split, phases 0, no meta tokens: merge the partial results inside the split kernel instead
 * of in a kernel of its own. The splits of a row run on one XCD (the launch sees to that), so the last of
 * its wavefronts to finish can pick the others' partials up from the shared L2 without any cache write-back;
 * same arithmetic and order as the merge kernel, same bits. Measured NOT faster on MI355X at 16..128 rows
 * (the hand-over chain at the end of the kernel costs what the second launch costs), hence opt-in. Needs the
 * workspace's first 64 KiB zeroed before its first use (see below). */
#define SB_DECODE_MERGE_IN_KERNEL 4

/* bf16/fp16 queries over a paged element cache with one query row per sequence, no key_lo and no meta rows
 * (the serving path) run the split as ONE stream of chunks per wavefront (swa_decode_stream.hip): a row
 * boundary inside a balanced run costs no pipeline restart, and nothing is fetched twice. This flag keeps such
 * calls on the per-segment kernels (swa_decode_mfma.hip), which serve every other case anyway (dense K/V,
 * row_seq, key_lo, meta rows, prefetch depths 2 and 3, the merge inside the kernel). Same results up to fp32
 * summation order. */
#define SB_DECODE_PER_SEGMENT 8

typedef struct sb_swa_decode_args {
  const void *q;   /* [num_rows, num_q_heads, head_size] */
  const void *k_cache;
  const void *v_cache;
  void *out;       /* [num_rows, num_q_heads, head_size] */
  float *lse;      /* optional */
  const int32_t *block_table; /* [num_seqs, block_table_stride] or NULL */
  const int64_t *kv_start;    /* dense mode: first row of each sequence, or NULL (= 0) */
  const int32_t *row_seq;     /* [num_rows] sequence of each query row, or NULL (= r) */
  const int32_t *seq_lens;    /* [num_rows] */
  const int32_t *key_lo;      /* [num_rows] or NULL */
  void *workspace;
  size_t workspace_bytes;
  int64_t num_rows;
  int32_t num_q_heads, num_kv_heads, head_size, block_size;
  int32_t window_left;
  int32_t max_seq_len; /* upper bound of seq_lens (host knowledge); sizes the split */
  int32_t n_split;     /* 0 = auto */
  int32_t dtype;
  int32_t phases;      /* 0 = split then merge; 1 = split kernel only; 2 = merge kernel only
                          (1 and 2 exist so a profiler can time the two kernels apart) */
  int32_t flags;       /* SB_DECODE_* bits */
  float scale;
  int64_t q_stride_row, q_stride_head;
  int64_t out_stride_row, out_stride_head;
  int64_t kv_stride_block, kv_stride_row, kv_stride_head;
  int64_t block_table_stride;
  /* Optional fused append (all three NULL = attention only). When set, row r's newest key
   * (index seq_lens[r]-1) has not been appended yet: its K/V rows are new_key[r] / new_value[r]
   * ([num_rows, num_kv_heads, head_size], strides below) and the call also stores them at
   * new_slot_mapping[r] (int64; < 0 = do not store), i.e. it does what reshape_and_cache_flash
   * (meta_attention.py:790-799) followed by the decode call (:965-981) do, in one launch.
   * Requires paged mode, one query row per sequence (row_seq NULL); k_cache/v_cache are
   * written. */
  const void *new_key;
  const void *new_value;
  const int64_t *new_slot_mapping;
  int64_t new_key_stride_row, new_key_stride_head;
  int64_t new_value_stride_row, new_value_stride_head;
  void *stream;
  /* Per-row INT8 cache (kv_quant = SB_KV_INT8): k_cache/v_cache hold int8 codes
   * [num_blocks, block_size, Hkv, 128] (kv strides in bytes), k_scale/v_scale the fp32 scales
   * [num_blocks, Hkv, block_size] that sb_kv_append_int8 wrote. Paged mode, q/out bf16 or fp16, fixed
   * split; the append is not fused (new_key etc. must be NULL: quantise and append first). */
  const float *k_scale;
  const float *v_scale;
  int32_t kv_quant;
  /* fp8 cache (kv_quant = SB_KV_FP8): k_cache/v_cache hold e4m3fn codes [num_blocks, block_size, Hkv, 128]
   * (kv strides in bytes), dequantised as code * k_scale_tensor / v_scale_tensor. Same restrictions as
   * the INT8 cache. */
  float k_scale_tensor, v_scale_tensor;
  /* Meta (sink) tokens, the query2/key2/value2 path of vllm_hymeta/attention/fa_kernel_metatoken.py:
   * 110-194: every query row also attends, without mask or window, to the meta_len rows of meta_k /
   * meta_v ([meta_len, num_kv_heads, 128] of dtype, strides in elements), the same rows for every
   * sequence. The reference runs a second attention and merges the two results by their log-sum-exp;
   * here the 32-row chunks of the meta rows are dealt round robin to the splits of each query row's
   * window and enter the same online softmax, so out and lse are those of ONE softmax over window
   * and meta keys (a row with an empty window attends to the meta rows alone). meta_len = 0 = off.
   * Fixed split only (rejected with SB_DECODE_BALANCED on the matrix-core kernels). fp32 queries and
   * SB_DECODE_FORCE_VALU take them in the vector kernel, whose wavefronts are dealt the meta rows 16 at a
   * time; soft cap / ALiBi: see below. Over a byte-code cache (kv_quant; bf16/fp16 queries only) the meta
   * rows are still elements of dtype: they are not quantised, and an fp8 cache's tensor scales do not
   * apply to them. */
  const void *meta_k;
  const void *meta_v;
  int32_t meta_len;
  int64_t meta_stride_row, meta_stride_head;
  /* Optional timing of the split kernel alone (both NULL = off): two hipEvent_t created with timing
   * enabled, attached to the kernel's own dispatch (hipExtLaunchKernel), i.e. recorded when that
   * kernel starts and when it ends, without any marker of their own in the stream. hipEventElapsedTime
   * between them is the kernel's duration as a kernel trace shows it. Fixed-split matrix-core kernel,
   * bf16/fp16 caches; ignored elsewhere. */
  void *profile_start_event;
  void *profile_stop_event;
  /* The two score options the backend passes on to flash-attn (meta_attention.py:665-690, :965-981
   * alibi_slopes=..., softcap=...): softcap > 0 turns every scaled score x into softcap * tanh(x / softcap);
   * alibi_slopes ([num_q_heads] fp32, NULL = off) adds -slope[h] * (query position - key index), the query
   * sitting at key index seq_lens[r]-1. Both are applied in front of the mask, the cap first. Any query
   * type (the fp32 vector kernel takes them too); over element, INT8 and fp8 caches.
   * Together with meta rows (any query type): the cap applies to their scores as to any other; their ALiBi term
   * is the one flash-attn gives them in the reference's second attention call
   * (fa_kernel_metatoken.py:169-188: all query rows of the call stacked as ONE sequence of
   * meta_bias_rows queries against the meta_len meta keys, causal=False), i.e. for query row r and meta
   * row j:  -slope[h] * |meta_bias_row0 + r + meta_len - meta_bias_rows - j|.  meta_bias_row0 is the
   * index of this call's row 0 in that stacked sequence (0 when the call holds all of its rows),
   * meta_bias_rows its length (0 = num_rows). */
  float softcap;
  const float *alibi_slopes;
  int64_t meta_bias_row0, meta_bias_rows;
} sb_swa_decode_args;

/* Split count the auto rule (n_split = 0) would use for these shapes: the one with the lowest estimated
 * duration, counting the rounds in which rows x splits workgroups pass over the CUs (one at a time per CU). */
int32_t sb_swa_decode_auto_split(int64_t num_rows, int32_t num_kv_heads, int32_t max_seq_len,
                                 int32_t window_left);
/* 1 if SB_DECODE_BALANCED is expected to be faster than the fixed split into n_split (>= 1) parts for rows
 * with these lengths, else 0. host_seq_lens: the step's seq_lens as a HOST array (the scheduler has them;
 * a caller without them can pass max_seq_len for every row: the balanced split adapts to the real lengths
 * on the device); no device access. */
int32_t sb_swa_decode_prefer_balanced(const int32_t *host_seq_lens, int64_t num_rows, int32_t window_left,
                                      int32_t n_split);

/* Bytes of workspace sb_swa_decode needs for a given split count (0 when n_split == 1). */
size_t sb_swa_decode_workspace_bytes(int64_t num_rows, int32_t num_q_heads, int32_t head_size,
                                     int32_t n_split);
int sb_swa_decode(const sb_swa_decode_args *args);

/* ------------------------------------------------------------------------------------
 * sb_swa_decode without any workspace from the caller and without any allocation.
 * No counterpart in the reference. It is for callers that cannot allocate device memory around
 * the call: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same arguments, kernels and results as sb_swa_decode (bit for bit), except that `workspace` /
 * `workspace_bytes` are ignored: the split-K partial results live in a device array of
 * SB_SWA_DECODE_STATIC_SCRATCH_BYTES that is part of the library image (every GPU the library runs
 * on holds its own copy from module load until the process ends). A call whose partials need more
 * (sb_swa_decode_workspace_bytes for its rows, heads and split count) is rejected with
 * SB_ERR_WORKSPACE before anything is launched. The call makes no hipMalloc / hipFree and calls no
 * allocating routine; the first call on a device looks the array's address up once
 * (hipGetSymbolAddress; make that call outside stream capture, with the device of the tensors
 * current on the calling thread).
 * All calls on one GPU share that GPU's array: calls on different streams of one GPU that overlap
 * in time race on the partials (calls on one stream are ordered and safe). Every partial a merge
 * reads has been written by the same call's split kernel, so nothing needs clearing between calls.
 * ------------------------------------------------------------------------------------ */
#define SB_SWA_DECODE_STATIC_SCRATCH_BYTES (8u << 20)
int sb_swa_decode_static(const sb_swa_decode_args *args);

/* ------------------------------------------------------------------------------------
 * GLA recurrent step(s) with in-place, slot-indexed state.
 * Replaces my_fused_recurrent_gla (vllm_hymeta/model_for_7B/my_fused_recurrent.py:9-153,
 * called from vllm_hymeta/model_for_7B/gla_attention.py:232) for T = 1, and
 * fla.ops.gla.fused_recurrent_gla as called from hf_7B_model/gla_attention.py:153 for T >= 1
 * (and fla's fused_chunk_gla as called from vllm_hymeta/model_for_7B/gla_attention.py:207-208:
 * the same recurrence over a prompt, final state handed to the slot cache).
 * Per (b, h), for t = 0..T-1:
 *     S  <- exp(g_t)[:,None] * S + k_t[:,None] * v_t[None,:]        (S is [dk, dv])
 *     o_t = sum_dk (q_t*scale)[:,None] * S                          (uses the updated S)
 * State of batch row b is state[slot_idx[b]] (slot_idx NULL = b); slot_idx[b] == -1 leaves
 * state and output of that row untouched (my_fused_recurrent.py:32-36). fp32 math; state
 * is read once and written once per call whatever T is. dk = dv = 128.
 *   q,k,v  [B, H, T, 128] dtype `dtype` (batch/head/time strides given)
 *   g      [B, H, T, 128] dtype `g_dtype` (log-space gate per key dim)
 *   state  [num_slots, H, 128, 128] dtype `state_dtype` (SB_F32 or SB_BF16)
 *   out    [B, H, T, 128] dtype `dtype`
 * ------------------------------------------------------------------------------------ */
#define SB_GLA_VECTOR_ONLY 1
#define SB_GLA_CHECK_GATES 2 /* matrix-core block form: count gates beyond its range (see flags, sb_gla_gate_range_hits) */
#define SB_GLA_PER_HEAD 4 /* shared states, matrix-core block form: one workgroup per query head (two launches), whatever the batch */
#define SB_GLA_GROUP_PASS 8 /* ... one workgroup per group of query heads (one launch), whatever the batch; default: by batch size */

typedef struct sb_gla_recurrent_args {
  const void *q, *k, *v, *g;
  void *state;
  void *out;
  const int32_t *slot_idx;
  int64_t batch;
  int32_t num_heads, seq_len, head_dim;
  int32_t dtype, g_dtype, state_dtype;
  float scale;
  int64_t q_stride_b, q_stride_h, q_stride_t;
  int64_t k_stride_b, k_stride_h, k_stride_t;
  int64_t v_stride_b, v_stride_h, v_stride_t;
  int64_t g_stride_b, g_stride_h, g_stride_t;
  int64_t out_stride_b, out_stride_h, out_stride_t;
  int64_t state_stride_slot, state_stride_head;
  int64_t num_slots; /* bound for documentation; slot_idx values are trusted */
  void *stream;
  /* Optional packed (varlen) form, the prefill loop of vllm_hymeta/model_for_7B/gla_attention.py:179-221
   * (one fused_chunk_gla call per request, state copied into the slot cache) as ONE launch: when
   * cu_seqlens ([batch+1] int32) is given, batch row b owns tokens cu_seqlens[b] .. cu_seqlens[b+1]-1 of
   * q/k/v/g/out laid out [total_tokens, H, 128]; the *_stride_b fields are ignored, the *_stride_t
   * fields are the token strides, and seq_len is only an upper bound of the row lengths. */
  const int32_t *cu_seqlens;
  /* SB_GLA_* bits. Calls of 32 steps or more, and every packed call, with bf16 q/k/v run the
   * recurrence 16 tokens at a time on the matrix cores (its exact block form; fp32 state, gate
   * scan and accumulation; bf16 operand rounding on the output path as in any bf16 GEMM).
   * SB_GLA_VECTOR_ONLY keeps such calls on the step-by-step fp32 kernel.
   * Gate range of the block form: inside a pair of blocks it forms exp(-(g_1 + .. + g_s)) per key dim, with
   * the exponent clamped at 80, so it is exact only while the gates of any 32 consecutive tokens sum to
   * more than -80 per key dim (|g| up to 2.5 per token, sustained; the model's log-sigmoid(x) / 16 gates
   * reach that only for x < -40). Beyond it near-diagonal q.k terms are under-weighted; the call itself
   * returns no error (it does not wait for the kernel); with SB_GLA_CHECK_GATES every such event adds to
   * a device counter that sb_gla_gate_range_hits reads (a build of the kernel of its own, 0-4 % slower). Callers whose gates can be that negative
   * set SB_GLA_VECTOR_ONLY, which has no such limit (fla's fused_chunk_gla, which this path replaces,
   * divides by the same cumulative decays inside its chunks). */
  int32_t flags;
  /* Shared states, 0 or 1 = off. The reference computes k, v and the gate for the 4 kv heads and
   * repeats them to the 28 query heads (hf_7B_model/gla_attention.py:147-149,
   * vllm_hymeta/model_for_7B/gla_attention.py:264-267), so the q_heads_per_state = 7 query heads of
   * a group carry bit-identical states as long as they start identical (they do: zeros). With
   * q_heads_per_state = G > 1, k, v, g and state have num_heads / G heads (query head h uses head
   * h / G of them), q and out keep num_heads heads, and every state is read and written once per
   * step for its whole group: the state traffic of a decode step drops G-fold, results unchanged.
   * Prompts on the matrix cores (the block form above) come in two shapes with the same bits: one workgroup
   * per query head, each carrying the recurrence for its own outputs (two ordered launches, the group's
   * first head stores the state), or one workgroup per group, which advances the state once and forms all
   * G outputs against it (vllm_hymeta/model_for_7B/gla_attention.py:264-267 "can be optimised later"); the
   * second where batch x (num_heads / G) >= 112 groups fill the machine by themselves, SB_GLA_PER_HEAD /
   * SB_GLA_GROUP_PASS to choose by hand.
   * num_heads must be a multiple of G, G <= 8. */
  int32_t q_heads_per_state;
  /* Optional timing of the decode-step kernel (one token, one state per head), as for sb_swa_decode. */
  void *profile_start_event;
  void *profile_stop_event;
} sb_gla_recurrent_args;

int sb_gla_recurrent(const sb_gla_recurrent_args *args);

/* Gate range check of the block form above. No counterpart in the reference (fla's kernel gives no such
 * signal). *hits = number of times the matrix-core GLA launches made with SB_GLA_CHECK_GATES on the current
 * device met gates beyond the range stated at `flags` (one per prompt, head, 32 key dims and pair of 16-token blocks concerned), since
 * the counter was last cleared; reset != 0 clears it. Waits for the device (a blocking copy): call it where a synchronisation is
 * acceptable, e.g. once after the prompts of a batch, not under stream capture. 0 hits = every block-form
 * result so far is exact in the sense stated there. */
int sb_gla_gate_range_hits(int64_t *hits, int32_t reset);

/* ------------------------------------------------------------------------------------
 * Block copy inside one device (copy-on-write of cache blocks).
 * Replaces ops.copy_blocks as called from meta_attention.py:115-126, for ONE cache
 * tensor half per call.  pairs = [num_pairs, 2] int64 (src block, dst block).
 * ------------------------------------------------------------------------------------ */
int sb_copy_blocks(void *cache, const int64_t *pairs, int64_t num_pairs, int64_t block_bytes,
                   int64_t stride_block_bytes, void *stream);

/* ------------------------------------------------------------------------------------
 * Dense sliding-window append for the HuggingFace-style cache.
 * Replaces the roll + slice-assign of hf_7B_model/cache.py:96-104: dst holds, per (b, h),
 * the last (keep) rows of src followed by the n new rows, in chronological order.
 * src/dst rows are [rows, D] planes addressed as plane p = b*H + h:
 *     src + p*src_stride_plane + (src_row0 + r)*D,  dst likewise. Byte copy, bit-exact.
 * Used by the cache's amortised compaction (one call per `capacity - window` appends).
 * ------------------------------------------------------------------------------------ */
typedef struct sb_window_shift_args {
  const void *src; /* old storage */
  void *dst;       /* new storage (must not overlap src rows being read) */
  const void *fresh; /* new rows [planes, n_new, D] with stride fresh_stride_plane / fresh_stride_row, may be NULL */
  int64_t planes;
  int64_t keep_rows, src_row0, dst_row0;
  int64_t n_new;
  int64_t row_bytes;
  int64_t src_stride_plane_bytes, dst_stride_plane_bytes;
  int64_t fresh_stride_plane_bytes, fresh_stride_row_bytes;
  void *stream;
} sb_window_shift_args;

int sb_window_shift(const sb_window_shift_args *args);

/* ------------------------------------------------------------------------------------
 * Causal sliding-window attention over many query tokens per sequence (prompt prefill,
 * chunked prefill over the paged cache, multi-token decode); bf16 / fp16, head_size 128,
 * GQA group size 1, 2, 4 or 7.
 * Replaces flash_attn_varlen_func as called from
 *   vllm_hymeta/attention/fa_kernel_metatoken.py:235-253 (via meta_attention.py:827-871,
 *   window_size = (window_left, 0), causal, block_table optional) and
 *   hf_7B_model/window_attention.py:186-204.
 * Query j of sequence s (row cu_seqlens_q[s] + j of q/out) sits at key position
 *   pos = seq_lens_k[s] - (cu_seqlens_q[s+1] - cu_seqlens_q[s]) + j
 * and attends keys i with max(0, pos - window_left) <= i <= pos (window_left < 0: all i <= pos),
 * further restricted to i >= key_lo[s] when key_lo is given; a query with no visible key gets zeros.
 * Keys of sequence s are addressed
 *   block_table != NULL: key i lives in block block_table[s*block_table_stride + i/block_size],
 *                        row i % block_size  (k, v = paged caches [blocks, block_size, Hkv, D]);
 *   block_table == NULL: row kv_start[s] + i of k / v  ([rows, Hkv, D]; kv_start NULL = 0).
 * The host supplies the tiling of the query axis: tile t covers queries
 *   tile_q0[t] .. tile_q0[t]+63 of sequence tile_seq[t] (clipped to the sequence's length);
 * every query must be covered by exactly one tile.
 * ------------------------------------------------------------------------------------ */
typedef struct sb_swa_prefill_args {
  const void *q;   /* [total_q, Hq, D] */
  const void *k;
  const void *v;
  void *out;       /* [total_q, Hq, D] */
  const int32_t *block_table; /* [S, block_table_stride] or NULL */
  const int64_t *kv_start;    /* [S] or NULL (dense addressing only) */
  const int32_t *key_lo;      /* [S] or NULL: keys below this index are invisible (left padding) */
  const int32_t *cu_seqlens_q; /* [S+1] */
  const int32_t *seq_lens_k;   /* [S] */
  const int32_t *tile_seq;     /* [num_tiles] */
  const int32_t *tile_q0;      /* [num_tiles] */
  int64_t num_tiles;
  int32_t num_q_heads, num_kv_heads, head_size, block_size;
  int32_t window_left;
  int32_t dtype;
  float scale;
  int64_t q_stride_row, q_stride_head;     /* elements */
  int64_t out_stride_row, out_stride_head;
  int64_t kv_stride_block, kv_stride_row, kv_stride_head; /* elements; block stride unused when dense;
                                                             a row stride of 16 MiB or more is rejected */
  int64_t block_table_stride;
  void *stream;
  float *lse;      /* optional, fp32 [total_q, Hq], natural log: log-sum-exp of each query's scaled scores,
                      the second result of _flash_attn_varlen_forward that fa_kernel_metatoken.py:254-257 merges on */
  /* byte-code paged caches, as for sb_swa_decode: kv_quant = SB_KV_INT8 with k_scale / v_scale, or
   * SB_KV_FP8 with k_scale_tensor / v_scale_tensor; k/v then hold codes and the kv strides are bytes.
   * Rows are dequantised (code * scale, rounded to dtype) on their way into the kernel's LDS stage. */
  const float *k_scale;
  const float *v_scale;
  int32_t kv_quant;
  float k_scale_tensor, v_scale_tensor;
  /* Meta (sink) tokens, as for sb_swa_decode (fa_kernel_metatoken.py:235-279: the varlen attention, a
   * second non-causal attention of all queries over k2/v2, and the log-sum-exp merge): every query
   * also attends, unmasked, to the meta_len rows of meta_k / meta_v ([meta_len, num_kv_heads, 128] of
   * dtype, strides in elements); their 32-row chunks are walked in front of each tile's window chunks,
   * inside the same softmax, and lse covers both. meta_len = 0 = off. Over a byte-code cache the meta
   * rows are still elements of dtype (not quantised, no scales). */
  const void *meta_k;
  const void *meta_v;
  int32_t meta_len;
  int64_t meta_stride_row, meta_stride_head;
  /* Score options as for sb_swa_decode (fa_kernel_metatoken.py:235-253 alibi_slopes=..., softcap=...): query j
   * of a sequence sits at key index seq_lens_k - query_len + j. Together with meta rows: as for
   * sb_swa_decode, the stacked sequence of fa_kernel_metatoken.py:258-275 being the call's packed query rows:
   * row t of q/out is its query meta_bias_row0 + t, and meta_bias_rows (required then: the kernel does not
   * know the total) is that sequence's length: the packed query rows plus the meta tokens' own queries. */
  float softcap;
  const float *alibi_slopes;
  int64_t meta_bias_row0, meta_bias_rows;
} sb_swa_prefill_args;

int sb_swa_prefill(const sb_swa_prefill_args *args);

/* ------------------------------------------------------------------------------------
 * Per-row symmetric INT8 K/V (W8ASpike/window_attention.py:183-186 with quantize_sym, :227-237):
 *   scale = clamp(max|row| / 127, 1e-5, 1e4); code = clamp(round_half_even(x / scale), -128, 127)
 * for every (token, kv head) row of head_size = 128 values. The reference re-quantises the whole
 * window at every step (and dequantises at once: "fake" quantisation); here a row is quantised
 * once, when it enters the cache, and stays 1 byte per value in HBM: half the bytes a decode
 * step reads. Codes and scales are bit-identical to quantize_sym's.
 *
 * sb_kv_append_int8: slot-mapped append (same slot_mapping contract as sb_kv_append).
 *   key, value      [num_tokens, num_kv_heads, 128] of dtype (bf16/fp16/fp32)
 *   k_cache, v_cache int8 [num_blocks, block_size, num_kv_heads, 128] (strides in bytes = elements)
 *   k_scale, v_scale fp32 [num_blocks, num_kv_heads, block_size] contiguous (head-major inside a
 *                   block: the 16 scales a 16-key tile of one head needs are one 64-byte run)
 * sb_quantize_sym: out = (code * scale) rounded to dtype, i.e. quantize_sym itself, for K/V that
 *   are attended to before they are cached (the prompt step); in == out is allowed.
 * ------------------------------------------------------------------------------------ */
typedef struct sb_kv_append_int8_args {
  const void *key;
  const void *value;
  void *k_cache;
  void *v_cache;
  float *k_scale;
  float *v_scale;
  const int64_t *slot_mapping;
  int64_t num_tokens;
  int32_t num_kv_heads, head_size, block_size, dtype;
  int64_t key_stride_token, key_stride_head;     /* elements */
  int64_t value_stride_token, value_stride_head;
  int64_t cache_stride_block, cache_stride_row, cache_stride_head; /* bytes */
  void *stream;
} sb_kv_append_int8_args;

int sb_kv_append_int8(const sb_kv_append_int8_args *args);

typedef struct sb_quantize_sym_args {
  const void *in;  /* [rows, heads, 128] */
  void *out;
  int64_t rows;
  int32_t heads, head_size, dtype;
  int64_t in_stride_row, in_stride_head;   /* elements */
  int64_t out_stride_row, out_stride_head;
  void *stream;
} sb_quantize_sym_args;

int sb_quantize_sym(const sb_quantize_sym_args *args);

/* ------------------------------------------------------------------------------------
 * fp8 (OCP e4m3fn) K/V with per-tensor scales: the kv_cache_dtype = "fp8" branch of
 *   vllm_hymeta/attention/meta_attention.py:790-812 (reshape_and_cache_flash with layer._k_scale /
 *   layer._v_scale; the cache tensor viewed as float8_e4m3fn).
 * code = e4m3fn(clamp(x / scale, -448, 448)), round to nearest even, NaN kept; value = code * scale.
 * sb_kv_append_fp8: slot-mapped append into byte caches [num_blocks, block_size, num_kv_heads, 128]
 *   (strides in bytes); same slot_mapping contract as sb_kv_append.
 * sb_fp8_round: out = e4m3fn(clamp(in / scale)) * scale rounded to dtype, row by row (rows of
 *   row_elems elements, a multiple of 8): what a tensor looks like after the fp8 round trip, for
 *   queries (scaled_fp8_quant at :806-811) and for K/V attended to before they are cached (:853-869).
 * sb_swa_decode reads such a cache with kv_quant = SB_KV_FP8 and k_scale_tensor / v_scale_tensor.
 * ------------------------------------------------------------------------------------ */
typedef struct sb_kv_append_fp8_args {
  const void *key;
  const void *value;
  void *k_cache;
  void *v_cache;
  const int64_t *slot_mapping;
  int64_t num_tokens;
  int32_t num_kv_heads, head_size, block_size, dtype;
  int64_t key_stride_token, key_stride_head;     /* elements */
  int64_t value_stride_token, value_stride_head;
  int64_t cache_stride_block, cache_stride_row, cache_stride_head; /* bytes */
  float k_scale, v_scale;
  void *stream;
} sb_kv_append_fp8_args;

int sb_kv_append_fp8(const sb_kv_append_fp8_args *args);

int sb_fp8_round(const void *in, void *out, int64_t rows, int64_t row_elems, int64_t in_stride_row,
                 int64_t out_stride_row, int32_t dtype, float scale, void *stream);

/* ------------------------------------------------------------------------------------
 * Merge of two attention results over disjoint key sets by their log-sum-exps, in place:
 *   lse' = lse - logsigmoid(lse - block_lse)
 *   out' = out - sigmoid(block_lse - lse) * (out - block_out)      (fp32, rounded once to dtype)
 * Replaces the TorchScript `_update_out_and_lse` of
 *   vllm_hymeta/attention/fa_kernel_metatoken.py:110-122
 * with which the window attention (out, lse) is combined with the attention of the same queries
 * over the cached meta tokens (block_out, block_lse) at :189 and :277. A side whose lse is -inf
 * (no visible key) contributes nothing; if both are -inf the row stays as it is.
 * out, block_out: [rows, heads, head_size] of dtype (bf16/fp16/fp32), inner dimension contiguous,
 * head_size a multiple of 8; lse, block_lse: fp32 [rows, heads] contiguous, natural log.
 * ------------------------------------------------------------------------------------ */
typedef struct sb_lse_merge_args {
  void *out;
  float *lse;
  const void *block_out;
  const float *block_lse;
  int64_t rows;
  int32_t heads, head_size, dtype;
  int64_t out_stride_row, out_stride_head;             /* elements */
  int64_t block_out_stride_row, block_out_stride_head;
  void *stream;
} sb_lse_merge_args;

int sb_lse_merge(const sb_lse_merge_args *args);

/* ------------------------------------------------------------------------------------
 * Device-side decode-step advance for the sliding-window paged cache: every sequence of
 * the batch takes one more token; seq_lens, slot_mapping and the window-ordered block
 * tables of the step are produced on the GPU, and the window bookkeeping (evict the
 * blocks that left the window, allocate the block a sequence grows into, LIFO free
 * stack, sequences in batch-row order) is done there too.
 * Window-aware analogue of ops.advance_step_flashattn as called from
 *   vllm_hymeta/attention/meta_attention.py:338-409 (which bumps seq_lens and looks the
 *   slot up in pre-grown block tables), so that consecutive decode steps - or a captured
 *   graph of them - need no host-side metadata rebuild.
 * State (device memory owned by the caller, updated in place):
 *   n_tokens [B] int64   tokens each sequence has seen
 *   lo, hi   [B] int32   lowest / highest resident logical block (hi < lo: none)
 *   ring     [B, ring_blocks] int32   physical id of logical block j at ring[b][j % ring_blocks]
 *   free_stack [num_blocks] int32, free_top [1] int32   free ids; the next allocation takes
 *                                                     free_stack[free_top - 1]
 * Outputs of the step:
 *   slot_mapping [B] int64, seq_lens [B] int32 (keys visible through the table, the new
 *   token included), block_tables [B, table_width] int32 (oldest resident block first,
 *   0 beyond the last), status [1] int32 (sticky; bit 0 = out of blocks, bit 1 = a
 *   sequence outgrew its ring; the caller reads it when it next synchronises).
 * A sequence that needs a block when the free stack is empty does not take its token: its slot is -1
 * (the step's append skips it), its seq_len counts the cached keys only, its token count stays, and no
 * block of another sequence is touched; its attention output of that step is meaningless. Callers that
 * run steps back to back (a replayed graph) must poll `status`.
 * ------------------------------------------------------------------------------------ */
typedef struct sb_window_advance_args {
  int64_t *n_tokens;
  int32_t *lo;
  int32_t *hi;
  int32_t *ring;
  int32_t *free_stack;
  int32_t *free_top;
  int64_t *slot_mapping;
  int32_t *seq_lens;
  int32_t *block_tables;
  int32_t *status;
  int64_t batch;
  int32_t ring_blocks, block_size, window_left, table_width, num_blocks;
  void *stream;
} sb_window_advance_args;

int sb_window_advance(const sb_window_advance_args *args);

/* ------------------------------------------------------------------------------------
 * Plain device-to-device streaming copy (non-temporal 16-byte lanes), `bytes` a multiple of
 * 16384. No counterpart in the reference: it is the measured bandwidth yardstick printed by
 * bench.py next to the kernels, and the launch of known size that the HBM byte counters
 * (FETCH_SIZE / WRITE_SIZE) are calibrated against.
 * ------------------------------------------------------------------------------------ */
int sb_stream_copy(void *dst, const void *src, int64_t bytes, void *stream);

/* ------------------------------------------------------------------------------------
 * Identity of the stream capture `stream` is part of: *id = the runtime's capture sequence number,
 * or 0 when the stream is not capturing. No counterpart in the reference (there the graph runner of
 * vLLM owns every buffer a captured step touches); the host layer uses it to give each captured graph
 * a split-K workspace of its own that no later call can replace or free. Returns 0 or the hipError_t.
 * ------------------------------------------------------------------------------------ */
int sb_stream_capture_id(void *stream, uint64_t *id);

#ifdef __cplusplus
}
#endif
#endif /* SBCACHE_H */
