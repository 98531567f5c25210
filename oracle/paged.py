"""Plain-Python/numpy model of the paged sliding-window KV cache bookkeeping.

TEST INFRASTRUCTURE: see oracle/__init__.py.

The reference delegates this bookkeeping to vLLM 0.10.0 (v0 block manager, model runner and
`vllm.attention.backends.utils`), which is not vendored in the reference tree; what the
reference's own files fix is the call pattern (vllm_hymeta/attention/meta_attention.py:474-494,
556-569, 790-799). The functions below restate that call pattern; the allocator policy
(LIFO free stack, evict-then-allocate per sequence in batch-row order) is this build's own
specification and is pinned by brute force in tests/test_oracle_paged.py.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

PAD_SLOT_ID = -1  # meta_attention.py:558 pads graph lanes with it; the append skips slot < 0


def kv_append(key: np.ndarray, value: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
              slot_mapping: Sequence[int]) -> None:
    """reshape_and_cache_flash as called at meta_attention.py:790-799, IN PLACE:
    cache[slot // bs, slot % bs, h, :] = key[t, h, :] for every token with slot >= 0.
    key/value [T, Hkv, D]; caches [nb, bs, Hkv, D]."""
    bs = k_cache.shape[1]
    for t, slot in enumerate(slot_mapping):
        slot = int(slot)
        if slot < 0:
            continue
        k_cache[slot // bs, slot % bs] = key[t]
        v_cache[slot // bs, slot % bs] = value[t]


def compute_slot_mapping_start_idx(is_prompt: bool, query_len: int, context_len: int,
                                   sliding_window: Optional[int]) -> int:
    """Call site meta_attention.py:489-491: prompt tokens older than the window are never
    cached."""
    start_idx = 0
    if is_prompt and sliding_window is not None:
        start_idx = max(0, query_len - sliding_window)
    return start_idx


def compute_slot_mapping(is_profile_run: bool, slot_mapping: List[int], seq_id, seq_len: int,
                         context_len: int, start_idx: int, block_size: int, block_tables: Dict) -> None:
    """Call site meta_attention.py:492-494: appends one slot per new token i in
    [context_len, seq_len): PAD for i < start_idx, else bt[i // bs] * bs + i % bs."""
    if is_profile_run:
        slot_mapping.extend([PAD_SLOT_ID] * seq_len)
        return
    padding_mask_len = max(0, start_idx - context_len)
    slot_mapping.extend([PAD_SLOT_ID] * padding_mask_len)
    block_table = block_tables[seq_id]
    for i in range(max(start_idx, context_len), seq_len):
        slot_mapping.append(int(block_table[i // block_size]) * block_size + i % block_size)


class WindowCacheModel:
    """Brute-force model of the window block manager: Python lists and dicts only.

    State per sequence: n tokens seen, resident logical blocks with their physical ids.
    One call = the new tokens of one sequence in one engine step (a prompt chunk, or one decode
    token), first new position p0 = n (window_left = wl, block_size = bs):
      1. evict    lo' = max(0, (p0 - wl) // bs); free the physical ids of resident logical
                  blocks < lo', lowest first, each pushed on top of the free stack. Nothing that
                  any query of this call can still see is evicted, so attention for the call
                  may read the cache after the append;
      2. store    token i is stored iff i >= start_idx (compute_slot_mapping_start_idx: for a
                  prompt attended over its in-flight K/V, tokens older than query_len - wl are
                  never cached, meta_attention.py:489-494; a chunked-prefill prompt, whose
                  queries read the paged cache, stores all); a stored token whose logical block i // bs has
                  no physical id pops the top of the free stack;
      3. slot     phys[i // bs] * bs + i % bs, PAD_SLOT_ID when not stored;
      4. view     block_table = phys[lo_res..hi] with lo_res the lowest resident logical block;
                  cache_seqlen = n_after - lo_res * bs (key index k of the view is absolute
                  position lo_res*bs + k; the last query sits at index cache_seqlen - 1)."""

    def __init__(self, num_blocks: int, block_size: int, window_left: int):
        self.bs = block_size
        self.wl = window_left
        self.free: List[int] = list(range(num_blocks - 1, -1, -1))  # pop() yields 0, 1, 2, ...
        self.seqs: Dict[int, dict] = {}

    def add_seq(self, seq_id: int) -> None:
        self.seqs[seq_id] = dict(n=0, phys={})  # phys: logical block -> physical id

    def free_seq(self, seq_id: int) -> None:
        s = self.seqs.pop(seq_id)
        for j in sorted(s["phys"]):
            self.free.append(s["phys"][j])

    def append_tokens(self, seq_id: int, count: int, is_prompt: bool, store_all: bool = False) -> List[int]:
        """Slots for `count` new tokens of one sequence (a prompt chunk or one decode token).
        store_all: a prompt chunk whose attention reads the paged cache keeps every token."""
        s = self.seqs[seq_id]
        p0 = s["n"]
        lo_new = max(0, (p0 - self.wl) // self.bs)
        for j in sorted(j for j in s["phys"] if j < lo_new):
            self.free.append(s["phys"].pop(j))
        start_idx = compute_slot_mapping_start_idx(is_prompt, count, p0, None if store_all else self.wl)
        slots = []
        for i in range(p0, p0 + count):
            if i < start_idx:
                slots.append(PAD_SLOT_ID)
                continue
            j = i // self.bs
            if j not in s["phys"]:
                if not self.free:
                    raise RuntimeError("out of blocks")
                s["phys"][j] = self.free.pop()
            slots.append(s["phys"][j] * self.bs + i % self.bs)
        s["n"] = p0 + count
        return slots

    def view(self, seq_id: int):
        """(block_table list, cache_seqlen, first resident position) as a kernel sees it now."""
        s = self.seqs[seq_id]
        if not s["phys"]:
            return [], 0, 0
        lo = min(s["phys"])
        hi = max(s["phys"])
        table = [s["phys"].get(j, 0) for j in range(lo, hi + 1)]
        return table, s["n"] - lo * self.bs, lo * self.bs

    def resident_blocks(self, seq_id: int) -> List[int]:
        return sorted(self.seqs[seq_id]["phys"])
