"""Model-runner slice for the sliding-window layers: turns a batch of sequences into the
per-step inputs the attention backend consumes (the part of vLLM's v0 model runner that feeds
vllm_hymeta/attention/meta_attention.py:435-608), on top of `WindowBlockManager`.

One block table / slot mapping is built per engine step and shared by every SWA layer, as in the
reference (each layer has its own KV tensor, all indexed by the same block ids).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .block_manager import LogicalTable, WindowBlockManager
from .meta_attention import Int8KVCache, MetaAttentionBackend, MetaAttentionMetadata, MetaAttentionMetadataBuilder


@dataclass
class SeqGroupData:
    """The per-sequence-group fields `MetaAttentionMetadataBuilder._add_seq_group` reads
    (meta_attention.py:445-453)."""
    is_prompt: bool
    seq_ids: List[int]
    input_tokens: List[List[int]]
    orig_seq_lens: List[int]
    seq_lens: List[int]
    query_lens: List[int]
    context_lens: List[int]
    curr_sliding_window_blocks: List[int]
    block_tables: Optional[Dict[int, "ResidentTable"]]
    prefix_cache_hit: bool = False
    multi_modal_placeholder_maps: Optional[dict] = None


class ResidentTable(LogicalTable):
    """A sequence's block table as the builder indexes it: `t[j]` by absolute logical block (slot
    mapping) and `t[-n:]` for the last n resident blocks (the window-bounded kernel table)."""

    def __len__(self) -> int:
        return int(self._mgr.hi[self._row]) + 1

    def __getitem__(self, j):
        if isinstance(j, slice):
            m, r = self._mgr, self._row
            lo, hi = int(m.lo[r]), int(m.hi[r])
            if j.stop is not None or j.step is not None or j.start is None or j.start >= 0:
                raise IndexError("only t[-n:] slices are supported")
            first = max(lo, hi + 1 + j.start)
            return m.ring[r, np.arange(first, hi + 1) % m.ring_blocks].tolist()
        return super().__getitem__(j)


@dataclass
class _Runner:
    device: torch.device
    pin_memory: bool = False
    graph_block_tables: Optional[object] = None


@dataclass
class _InputBuilder:
    runner: _Runner
    sliding_window: Optional[int]
    block_size: int
    chunked_prefill_enabled: bool
    inter_data_list: List[SeqGroupData] = field(default_factory=list)


class SwaCacheRunner:
    """Owns the block manager and the per-layer paged KV tensors; builds step metadata."""

    def __init__(self, num_layers: int, num_blocks: int, block_size: int, window_left: int, num_kv_heads: int,
                 head_size: int, dtype: torch.dtype, device, max_seqs: int, max_chunk_tokens: int = 0,
                 kv_quant: Optional[str] = None):
        """kv_quant="int8": every layer's cache is an Int8KVCache (codes + per-row scales) instead of a `dtype` tensor."""
        self.device = torch.device(device)
        self.block_size, self.window_left = block_size, window_left
        self.manager = WindowBlockManager(num_blocks, block_size, window_left, max_seqs, max_chunk_tokens)
        shape = MetaAttentionBackend.get_kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size)
        if kv_quant == "int8":
            self.kv_caches = [Int8KVCache.allocate(num_blocks, block_size, num_kv_heads, head_size, self.device)
                              for _ in range(num_layers)]
        elif kv_quant is None:
            self.kv_caches = [torch.zeros(shape, dtype=dtype, device=self.device) for _ in range(num_layers)]
        else:
            raise ValueError(f"kv_quant {kv_quant!r} (None or 'int8')")

    def add_seq(self, seq_id) -> None:
        self.manager.add_seq(seq_id)

    def free_seq(self, seq_id) -> None:
        self.manager.free_seq(seq_id)

    def build_step(self, prompts: Sequence[Tuple[int, int]], decodes: Sequence[int],
                   chunked_prefill: bool = False) -> MetaAttentionMetadata:
        """`prompts` = (seq_id, number of new prompt tokens); `decodes` = seq ids taking one token each, or
        (seq_id, n) pairs for decoding sequences that take n query tokens in this step (speculative /
        multi-token decode, the `max_decode_query_len > 1` branch of meta_attention.py:924-953).
        Advances the block manager (eviction, allocation) and returns the step's metadata with
        tokens laid out [prompt tokens | decode tokens]."""
        mgr, bs = self.manager, self.block_size
        # chunked prefill reads its keys back from the paged cache, so every prompt token is stored
        ib = _InputBuilder(_Runner(self.device), None if chunked_prefill else self.window_left, bs, chunked_prefill)
        seq_lens: List[int] = []
        query_lens: List[int] = []
        # the manager is advanced here, the builder recomputes the same slots from the tables
        for sid, n_new in prompts:
            r = mgr.row_of(sid)
            ctx = int(mgr.n_tokens[r])
            mgr.append_tokens(sid, n_new, True, store_all=chunked_prefill, want_slots=False)
            total = ctx + n_new
            first = int(mgr.lo[r]) * bs if mgr.hi[r] >= mgr.lo[r] else 0
            paged = chunked_prefill
            view_len = total - first if paged else total
            ib.inter_data_list.append(SeqGroupData(
                is_prompt=True, seq_ids=[sid], input_tokens=[[0] * n_new], orig_seq_lens=[total],
                seq_lens=[view_len], query_lens=[n_new], context_lens=[ctx],
                curr_sliding_window_blocks=[max(int(mgr.hi[r] - mgr.lo[r]) + 1, 0)],
                block_tables={sid: ResidentTable(mgr, r)}))
            seq_lens.append(view_len)
            query_lens.append(n_new)
        decodes = [d if isinstance(d, tuple) else (d, 1) for d in decodes]
        if decodes and all(n == 1 for _, n in decodes):
            mgr.decode_step([sid for sid, _ in decodes])
        else:
            for sid, n in decodes:      # same policy, one sequence after the other in batch-row order
                mgr.append_tokens(sid, n, False, want_slots=False)
        for sid, n in decodes:
            r = mgr.row_of(sid)
            total = int(mgr.n_tokens[r])
            view_len = total - int(mgr.lo[r]) * bs
            ib.inter_data_list.append(SeqGroupData(
                is_prompt=False, seq_ids=[sid], input_tokens=[[0] * n], orig_seq_lens=[total], seq_lens=[view_len],
                query_lens=[n], context_lens=[total - n],
                curr_sliding_window_blocks=[int(mgr.hi[r] - mgr.lo[r]) + 1],
                block_tables={sid: ResidentTable(mgr, r)}))
            seq_lens.append(view_len)
            query_lens.append(n)
        builder = MetaAttentionMetadataBuilder(ib)
        builder.prepare()
        return builder.build(seq_lens, query_lens, -1, len(seq_lens))
