// Kernel parameter block shared by the two split kernels (VALU and matrix-core) and the merge.
#pragma once
#include <stdint.h>
#include "common.h"
#ifndef SB_BALANCED_T
#define SB_BALANCED_T 3
#endif

namespace sb {

// Arrival counters of the in-kernel merge live in the first kMergeCounterBytes of the split-K workspace; the
// last of them is a sticky fault word (set if contributors to one merge ran on different XCDs).
constexpr int kMergeCounterBytes = 64 << 10;
constexpr int kMergeCounters = kMergeCounterBytes / 4 - 1;
constexpr int kMergeFaultWord = kMergeCounterBytes / 4 - 1;

// Balanced split of the per-segment kernel (swa_decode_mfma.hip): on the common chunk axis every non-empty row
// is preceded by this many virtual chunks. A workgroup of that kernel whose run crosses into a new row drains
// and refills its load pipeline there (a round trip to memory with nothing in flight); the virtual chunks
// charge that to its run, so it gets fewer real chunks than a workgroup that stays inside one row. That split
// kernel and its merge kernel share it. (The stream kernel crosses rows without a drain and has none.)
constexpr int kBalancedRowStartChunks = SB_BALANCED_T;

struct DecodeParams {
  const char *q;
  const char *k;
  const char *v;
  char *out;
  float *lse;
  const int32_t *block_table;
  const int64_t *kv_start;
  const int32_t *row_seq;
  const int32_t *seq_lens;
  const int32_t *key_lo;
  float *ws_acc;  // [rows, Hq, n_split, 128]
  float *ws_ml;   // [rows, Hq, n_split, 2]
  int32_t *ws_rows;  // balanced split, stream kernel: per row the first and last run (workgroup) holding a partial of it
  int Hq, block_size, window_left, n_split;
  int rows, n_wg;  // balanced split: query rows, workgroups per kv-head group (0 = fixed split)
  // Merge inside the split kernel (matrix-core fixed split): arrival counters [rows, Hkv], zero before and after
  // every launch, and the number of kv heads; null = the merge is a kernel of its own.
  int *merge_counter;
  int Hkv;
  float scale_log2;
  int64_t q_sr, q_sh, o_sr, o_sh;  // elements
  int64_t kv_sb, kv_sr, kv_sh;     // bytes
  int64_t bt_stride;
  // fused append (matrix-core kernel only): this step's key/value rows and their cache slots
  const char *new_k;
  const char *new_v;
  const int64_t *slot_mapping;
  int64_t nk_st, nk_sh, nv_st, nv_sh;  // bytes
  // INT8 cache: per-row scales [num_blocks, Hkv, block_size]
  const float *k_scale;
  const float *v_scale;
  float kv_out_scale;  // multiplies the result (fp8 cache: the V tensor scale; else 1)
  // Meta tokens (matrix-core fixed split only): meta_len rows [meta_len, Hkv, 128] of the query's type every
  // query row also attends to, without mask; meta_len = 0 = none
  const char *meta_k;
  const char *meta_v;
  int meta_len;
  int64_t meta_sr, meta_sh;  // bytes
  // Over a byte-code cache the meta rows are still elements: their scores and probabilities are multiplied by
  // these so that the scales folded into scale_log2 and kv_out_scale (fp8 cache) cancel for them; else 1.
  float meta_k_mult, meta_v_mult;
  // ALiBi term of meta row j for query row r: -slope * |meta_bias_off + r - j|, meta_bias_off = row0 + meta_len - rows
  // (the position flash-attn gives row r of the reference's stacked second attention)
  int meta_bias_off;
  // soft cap / ALiBi: applied to every raw score in front of the mask
  ScoreOptions opt;
  int D;  // head size (vector kernel and its merge; the matrix-core kernels are built for 128)
  int group_parts;  // vector kernel: workgroups that share a kv head (each takes its share of the group's query heads)
};

}  // namespace sb
