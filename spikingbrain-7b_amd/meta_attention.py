"""Attention backend for the sliding-window layers over the paged KV cache: drop-in for
vllm_hymeta/attention/meta_attention.py (backend / metadata / builder / impl).

Class names, method names, argument order, error types and the in-place `output` contract follow
the reference file; the kernels behind `forward` are libsbcache's (append, window-bounded paged
attention). vLLM itself is not a dependency: the few vLLM types the reference file leans on are
duck-typed (`input_builder`, `inter_data`, `layer`) or restated here (`AttentionType`).
"""
from __future__ import annotations

from collections import defaultdict
from dataclasses import dataclass
from itertools import accumulate
from typing import Any, Dict, List, Optional, Tuple, Type

import torch

from . import ops
from .block_manager import PAD_SLOT_ID, SlotBuffer, compute_slot_mapping, compute_slot_mapping_start_idx


class AttentionType:
    """String constants of vLLM's attention kinds (compared by value in the reference)."""
    DECODER = "decoder"
    ENCODER = "encoder"
    ENCODER_ONLY = "encoder_only"
    ENCODER_DECODER = "encoder_decoder"


_QUANTIZED_KV = ("fp8", "fp8_e4m3", "fp8_e5m2", "int8")


class CommonAttentionState:
    """Minimal per-runner attention state (the reference returns vLLM's class of this name,
    meta_attention.py:77-79); graph capture bookkeeping stays with the caller."""

    def __init__(self, runner=None):
        self.runner = runner

    def begin_forward(self, model_input) -> None:
        return None


class MetaAttentionBackend:
    """meta_attention.py:53-126."""

    accept_output_buffer: bool = True

    @staticmethod
    def get_supported_head_sizes() -> List[int]:
        """The reference's list (meta_attention.py:57-59: what flash-attn builds). The matrix-core and byte-code
        kernels here are built for head_dim 128, the 7B model's; the other sizes run every piece of a step on the
        vector kernel (one row per query token), with element caches only."""
        return [32, 64, 96, 128, 160, 192, 224, 256]

    @staticmethod
    def get_name() -> str:
        return "META_FLASH_ATTN"

    @staticmethod
    def get_impl_cls() -> Type["MetaAttentionImpl"]:
        return MetaAttentionImpl

    @staticmethod
    def get_metadata_cls() -> Type["MetaAttentionMetadata"]:
        return MetaAttentionMetadata

    @staticmethod
    def get_builder_cls() -> Type["MetaAttentionMetadataBuilder"]:
        return MetaAttentionMetadataBuilder

    @staticmethod
    def get_state_cls() -> Type["CommonAttentionState"]:
        return CommonAttentionState

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int) -> Tuple[int, ...]:
        if block_size % 16 != 0 or block_size < 16:
            raise ValueError(f"Invalid block size {block_size}. Must be a multiple of 16 and at least 16.")
        return (2, num_blocks, block_size, num_kv_heads, head_size)

    @staticmethod
    def swap_blocks(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor, scr_to_dst: torch.Tensor) -> None:
        """Move whole blocks between two cache tensors (device<->host or device<->device);
        scr_to_dst is [n, 2] (source block, destination block). Block-granular async copies on
        the current stream, K half then V half (meta_attention.py:94-112)."""
        pairs = scr_to_dst.tolist()
        if isinstance(src_kv_cache, Int8KVCache):
            tensors = ((src_kv_cache.codes, dst_kv_cache.codes), (src_kv_cache.scales, dst_kv_cache.scales))
        else:
            tensors = ((src_kv_cache, dst_kv_cache),)
        for src_t, dst_t in tensors:
            for half in (0, 1):
                src, dst = src_t[half], dst_t[half]
                for s, d in pairs:
                    dst[d].copy_(src[s], non_blocking=True)

    @staticmethod
    def copy_blocks(kv_caches: List[torch.Tensor], src_to_dists: torch.Tensor) -> None:
        """Copy-on-write block copies inside every layer's cache (meta_attention.py:114-126)."""
        for kv_cache in kv_caches:
            halves = (kv_cache.codes, kv_cache.scales) if isinstance(kv_cache, Int8KVCache) else (kv_cache,)
            for t in halves:
                ops.copy_blocks(t[0], src_to_dists)
                ops.copy_blocks(t[1], src_to_dists)


class Int8KVCache:
    """One layer's paged K/V in per-row INT8 form: `codes` int8 [2, num_blocks, block_size, Hkv, D] and
    `scales` fp32 [2, num_blocks, Hkv, block_size] (quantize_sym of W8ASpike/window_attention.py:227-237
    applied once per row, at append time). Pass it where the bf16 `kv_cache` tensor goes."""

    def __init__(self, codes: torch.Tensor, scales: torch.Tensor):
        if codes.dtype != torch.int8 or codes.dim() != 5 or codes.shape[0] != 2:
            raise ValueError("codes must be int8 [2, num_blocks, block_size, num_kv_heads, head_size]")
        _, nb, bs, hkv, _ = codes.shape
        if scales.dtype != torch.float32 or tuple(scales.shape) != (2, nb, hkv, bs):
            raise ValueError("scales must be float32 [2, num_blocks, num_kv_heads, block_size]")
        self.codes, self.scales = codes, scales

    @classmethod
    def allocate(cls, num_blocks: int, block_size: int, num_kv_heads: int, head_size: int, device) -> "Int8KVCache":
        MetaAttentionBackend.get_kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size)   # validates
        return cls(*ops.alloc_int8_kv_cache(num_blocks, block_size, num_kv_heads, head_size, device))

    def numel(self) -> int:
        return self.codes.numel()

    @property
    def device(self):
        return self.codes.device


@dataclass
class MetaAttentionMetadata:
    """meta_attention.py:128-336. Token layout: [prefill tokens | decode tokens]."""
    num_prefills: int
    num_prefill_tokens: int
    num_decode_tokens: int
    slot_mapping: Optional[torch.Tensor]
    seq_lens: Optional[List[int]]
    seq_lens_tensor: Optional[torch.Tensor]
    max_prefill_seq_len: int
    max_decode_seq_len: int
    context_lens_tensor: Optional[torch.Tensor]
    block_tables: Optional[torch.Tensor]
    use_cuda_graph: bool
    max_query_len: Optional[int] = None
    max_decode_query_len: Optional[int] = None
    query_start_loc: Optional[torch.Tensor] = None
    seq_start_loc: Optional[torch.Tensor] = None
    multi_modal_placeholder_index_maps: Optional[Dict[str, Any]] = None
    enable_kv_scales_calculation: bool = True
    _cached_prefill_metadata: Optional["MetaAttentionMetadata"] = None
    _cached_decode_metadata: Optional["MetaAttentionMetadata"] = None
    encoder_seq_lens: Optional[List[int]] = None
    encoder_seq_lens_tensor: Optional[torch.Tensor] = None
    encoder_seq_start_loc: Optional[torch.Tensor] = None
    max_encoder_seq_len: Optional[int] = None
    num_encoder_tokens: Optional[int] = None
    cross_slot_mapping: Optional[torch.Tensor] = None
    cross_block_tables: Optional[torch.Tensor] = None
    # Not in the reference's metadata: host copies of the per-sequence query and key counts (the
    # builder has them as Python ints anyway). With them the many-query kernel lays out its 64-token
    # tiles without reading a device tensor back; without them every query token runs as one row of
    # the single-query kernel.
    query_lens: Optional[List[int]] = None
    host_seq_lens: Optional[List[int]] = None
    _prefill_plan: Any = None
    _decode_balanced: Any = None     # split policy of this step's decode launch, decided once for all layers

    def prefill_plan(self, device) -> Any:
        """Tile layout of this (sub)step for ops.swa_prefill_attention, built once and shared by
        every layer; None when the host lengths are not known."""
        lens_k = self.seq_lens if self.seq_lens is not None else self.host_seq_lens
        if self.query_lens is None or lens_k is None:
            return None
        if self._prefill_plan is None:
            n = len(self.query_lens)
            self._prefill_plan = ops.PrefillPlan(self.query_lens, list(lens_k[:n]), device)
        return self._prefill_plan

    @property
    def is_all_encoder_attn_metadata_set(self) -> bool:
        return (self.encoder_seq_lens is not None and self.encoder_seq_lens_tensor is not None
                and self.max_encoder_seq_len is not None)

    @property
    def is_all_cross_attn_metadata_set(self) -> bool:
        return (self.is_all_encoder_attn_metadata_set and self.cross_slot_mapping is not None
                and self.cross_block_tables is not None)

    @property
    def prefill_metadata(self) -> Optional["MetaAttentionMetadata"]:
        if self.num_prefills == 0:
            return None
        if self._cached_prefill_metadata is not None:
            return self._cached_prefill_metadata
        assert (self.seq_lens is not None) or (self.encoder_seq_lens is not None)
        assert (self.seq_lens_tensor is not None) or (self.encoder_seq_lens_tensor is not None)
        n, nt = self.num_prefills, self.num_prefill_tokens

        def head(t, k):
            return None if t is None else t[:k]

        self._cached_prefill_metadata = MetaAttentionMetadata(
            num_prefills=n, num_prefill_tokens=nt, num_decode_tokens=0,
            slot_mapping=head(self.slot_mapping, nt),
            multi_modal_placeholder_index_maps=self.multi_modal_placeholder_index_maps,
            enable_kv_scales_calculation=self.enable_kv_scales_calculation,
            seq_lens=head(self.seq_lens, n), seq_lens_tensor=head(self.seq_lens_tensor, n),
            max_query_len=self.max_query_len, max_prefill_seq_len=self.max_prefill_seq_len,
            max_decode_query_len=0, max_decode_seq_len=0,
            query_start_loc=head(self.query_start_loc, n + 1), seq_start_loc=head(self.seq_start_loc, n + 1),
            context_lens_tensor=head(self.context_lens_tensor, n), block_tables=head(self.block_tables, n),
            use_cuda_graph=False,
            encoder_seq_lens=self.encoder_seq_lens, encoder_seq_lens_tensor=self.encoder_seq_lens_tensor,
            encoder_seq_start_loc=self.encoder_seq_start_loc, max_encoder_seq_len=self.max_encoder_seq_len,
            cross_slot_mapping=self.cross_slot_mapping, cross_block_tables=self.cross_block_tables,
            query_lens=head(self.query_lens, n), host_seq_lens=head(self.seq_lens, n))
        return self._cached_prefill_metadata

    @property
    def decode_metadata(self) -> Optional["MetaAttentionMetadata"]:
        if self.num_decode_tokens == 0:
            return None
        if self._cached_decode_metadata is not None:
            return self._cached_decode_metadata
        assert (self.seq_lens_tensor is not None) or (self.encoder_seq_lens_tensor is not None)
        n, nt = self.num_prefills, self.num_prefill_tokens

        def tail(t, k):
            return None if t is None else t[k:]

        self._cached_decode_metadata = MetaAttentionMetadata(
            num_prefills=0, num_prefill_tokens=0, num_decode_tokens=self.num_decode_tokens,
            slot_mapping=tail(self.slot_mapping, nt),
            multi_modal_placeholder_index_maps=None, enable_kv_scales_calculation=True,
            seq_lens=None, seq_lens_tensor=tail(self.seq_lens_tensor, n),
            max_decode_query_len=self.max_decode_query_len, max_query_len=self.max_query_len,
            max_prefill_seq_len=0, max_decode_seq_len=self.max_decode_seq_len,
            # [3 prefills | 6 decodes], query_start_loc [.., 3, 9] -> [0, 6]
            query_start_loc=(self.query_start_loc[n:] - self.query_start_loc[n])
            if self.query_start_loc is not None else None,
            seq_start_loc=tail(self.seq_start_loc, n),
            context_lens_tensor=None, block_tables=tail(self.block_tables, n),
            use_cuda_graph=self.use_cuda_graph,
            encoder_seq_lens=self.encoder_seq_lens, encoder_seq_lens_tensor=self.encoder_seq_lens_tensor,
            encoder_seq_start_loc=self.encoder_seq_start_loc, max_encoder_seq_len=self.max_encoder_seq_len,
            cross_slot_mapping=self.cross_slot_mapping, cross_block_tables=self.cross_block_tables,
            query_lens=tail(self.query_lens, n),
            host_seq_lens=tail(self.seq_lens if self.seq_lens is not None else self.host_seq_lens, n))
        return self._cached_decode_metadata


class MetaAttentionMetadataBuilder:
    """meta_attention.py:411-608. `input_builder` is duck-typed: it carries `runner` (with `device`,
    `pin_memory`, optional `graph_block_tables`), `sliding_window`, `block_size`, `inter_data_list`
    and `chunked_prefill_enabled`; each inter_data has the fields the reference zips over (:445-453)."""

    def __init__(self, input_builder):
        self.input_builder = input_builder
        self.runner = input_builder.runner
        self.sliding_window = input_builder.sliding_window
        self.block_size = input_builder.block_size

    def prepare(self):
        self.slot_mapping = SlotBuffer()   # the reference's List[int], kept as numpy pieces
        self.prefill_seq_lens: List[int] = []
        self.context_lens: List[int] = []
        self.block_tables: List[List[int]] = []
        self.curr_seq_lens: List[int] = []
        self.multimodal_placeholder_maps: Dict[str, Any] = defaultdict(list)
        self.num_prefills = 0
        self.num_prefill_tokens = 0
        self.num_decode_tokens = 0
        self.has_prefix_cache_hit = False

    def _add_seq_group(self, inter_data, chunked_prefill_enabled: bool, prefix_cache_hit: bool):
        """Per sequence: context length, window-bounded block table, slot mapping (:435-494)."""
        is_prompt = inter_data.is_prompt
        block_tables = inter_data.block_tables
        for (seq_id, token_len, seq_len, curr_seq_len, query_len, context_len, curr_sliding_window_block) in zip(
                inter_data.seq_ids, [len(t) for t in inter_data.input_tokens], inter_data.orig_seq_lens,
                inter_data.seq_lens, inter_data.query_lens, inter_data.context_lens,
                inter_data.curr_sliding_window_blocks):
            self.context_lens.append(context_len)
            if is_prompt:
                self.num_prefills += 1
                self.num_prefill_tokens += token_len
                self.prefill_seq_lens.append(seq_len)
            else:
                self.num_decode_tokens += query_len
                self.curr_seq_lens.append(curr_seq_len)

            block_table = []
            if prefix_cache_hit:
                block_table = block_tables[seq_id]
            elif (chunked_prefill_enabled or not is_prompt) and block_tables is not None:
                if curr_sliding_window_block == 0:
                    block_table = block_tables[seq_id]
                else:
                    block_table = block_tables[seq_id][-curr_sliding_window_block:]
            self.block_tables.append(list(block_table))

            is_profile_run = block_tables is None or all(len(t) == 0 for t in block_tables.values())
            start_idx = compute_slot_mapping_start_idx(is_prompt, query_len, context_len, self.sliding_window)
            compute_slot_mapping(is_profile_run, self.slot_mapping, seq_id, seq_len, context_len, start_idx,
                                 self.block_size, inter_data.block_tables)

    def _get_graph_runner_block_tables(self, num_seqs: int, block_tables: List[List[int]]) -> torch.Tensor:
        """Fill the runner's persistent [max_batch, max_blocks] numpy table and ship it (:496-519)."""
        max_batch_size, max_blocks = self.runner.graph_block_tables.shape
        assert max_batch_size >= num_seqs
        graph_block_tables = self.runner.graph_block_tables[:num_seqs]
        for i, block_table in enumerate(block_tables):
            if block_table:
                n = min(len(block_table), max_blocks)
                graph_block_tables[i, :n] = block_table[:n]
        return torch.from_numpy(graph_block_tables).to(device=self.runner.device, non_blocking=True)

    def build(self, seq_lens: List[int], query_lens: List[int], cuda_graph_pad_size: int, batch_size: int):
        """Device-side metadata for one engine step (:521-608)."""
        prefix_cache_hit = any(d.prefix_cache_hit for d in self.input_builder.inter_data_list)
        for inter_data in self.input_builder.inter_data_list:
            self._add_seq_group(inter_data, self.input_builder.chunked_prefill_enabled, prefix_cache_hit)

        device = self.runner.device
        use_captured_graph = cuda_graph_pad_size != -1
        max_query_len = max(query_lens)
        decode_query_lens = query_lens[self.num_prefills:]
        max_decode_query_len = max(decode_query_lens) if len(decode_query_lens) > 0 else 1
        max_prefill_seq_len = max(self.prefill_seq_lens, default=0)
        max_decode_seq_len = max(self.curr_seq_lens, default=0)
        num_decode_tokens = self.num_decode_tokens
        query_start_loc = list(accumulate(query_lens, initial=0))
        seq_start_loc = list(accumulate(seq_lens, initial=0))

        num_seqs = len(seq_lens)
        if use_captured_graph:
            self.slot_mapping.extend([PAD_SLOT_ID] * cuda_graph_pad_size)
            self.block_tables.extend([[] for _ in range(cuda_graph_pad_size)])
            num_decode_tokens = batch_size - self.num_prefill_tokens
            block_tables = self._get_graph_runner_block_tables(num_seqs, self.block_tables)
        else:
            width = max((len(t) for t in self.block_tables), default=0)
            padded = [t + [0] * (width - len(t)) for t in self.block_tables]
            block_tables = torch.tensor(padded, dtype=torch.int32).reshape(len(padded), width).to(device)
        assert max_query_len > 0, "query_lens: {}".format(query_lens)
        assert device is not None

        pin = bool(getattr(self.runner, "pin_memory", False)) and torch.device(device).type == "cuda"

        def h2d(data, dtype):
            if isinstance(data, SlotBuffer):
                t = torch.from_numpy(data.array()).to(dtype)
                return (t.pin_memory() if pin else t).to(device, non_blocking=True)
            return torch.tensor(data, dtype=dtype, pin_memory=pin).to(device, non_blocking=True)

        return MetaAttentionMetadata(
            num_prefills=self.num_prefills,
            slot_mapping=h2d(self.slot_mapping, torch.long),
            num_prefill_tokens=self.num_prefill_tokens,
            num_decode_tokens=num_decode_tokens,
            seq_lens=seq_lens,
            multi_modal_placeholder_index_maps={},
            enable_kv_scales_calculation=True,
            seq_lens_tensor=h2d(seq_lens, torch.int),
            max_query_len=max_query_len,
            max_decode_query_len=max_decode_query_len,
            max_prefill_seq_len=max_prefill_seq_len,
            max_decode_seq_len=max_decode_seq_len,
            query_start_loc=h2d(query_start_loc, torch.int32),
            seq_start_loc=h2d(seq_start_loc, torch.int32),
            context_lens_tensor=h2d(self.context_lens, torch.int),
            block_tables=block_tables,
            use_cuda_graph=use_captured_graph,
            query_lens=list(query_lens),
        )


class MetaAttentionImpl:
    """meta_attention.py:611-982.

    Token layout [prefill_0 .. prefill_N-1 | decode_0 .. decode_M-1 (| graph padding)].
    `sliding_window` is the window INCLUDING the current token; keys visible to a query are
    itself and the `sliding_window - 1` before it (:671-672; the 7B model passes W + 1,
    vllm_hymeta/model_for_7B/modeling_gla_swa.py:200, so window_left = W)."""

    def __init__(
        self,
        num_heads: int,
        head_size: int,
        scale: float,
        num_kv_heads: int,
        alibi_slopes: Optional[List[float]],
        sliding_window: Optional[int],
        kv_cache_dtype: str,
        blocksparse_params: Optional[Dict[str, Any]] = None,
        logits_soft_cap: Optional[float] = None,
        attn_type: str = AttentionType.DECODER,
        kv_sharing_target_layer_name: Optional[str] = None,
        use_irope: bool = False,
        num_meta_tokens: int = 128,
    ):
        if kv_sharing_target_layer_name is not None:
            raise NotImplementedError("KV sharing is not supported in V0 MetaAttention.")
        if blocksparse_params is not None:
            raise ValueError("MetaAttention does not support blocksparse attention.")
        self.num_heads = num_heads
        self.head_size = head_size
        self.scale = float(scale)
        self.num_kv_heads = num_kv_heads
        # (:665-670) one slope per query head, kept as an fp32 tensor and handed to the kernels as it is
        if alibi_slopes is not None:
            alibi_slopes = torch.tensor(alibi_slopes, dtype=torch.float32)
            if alibi_slopes.shape != (num_heads,):
                raise ValueError(f"alibi_slopes must hold one slope per query head ({num_heads})")
        self.alibi_slopes = alibi_slopes
        self.sliding_window = ((sliding_window - 1, 0) if sliding_window is not None else (-1, -1))
        self.kv_cache_dtype = kv_cache_dtype
        self.num_meta_tokens = num_meta_tokens
        # "fp8" / "fp8_e4m3": the cache tensor holds e4m3fn codes (uint8 or float8_e4m3fn, as the reference
        # views it at :801-803) with the layer's per-tensor scales. (An INT8 cache is not a dtype string
        # but an Int8KVCache object passed as kv_cache.)
        if kv_cache_dtype in ("fp8_e5m2", "int8") or (kv_cache_dtype.startswith("fp8")
                                                       and kv_cache_dtype not in ("fp8", "fp8_e4m3")):
            raise NotImplementedError(
                f"MetaAttention does not support {self.kv_cache_dtype} kv-cache on this device "
                "(fp8 means e4m3fn here).")
        if logits_soft_cap is None:
            # (:686-690) in flash-attn a soft cap of 0 means no soft cap; the kernels here read it the same way
            logits_soft_cap = 0
        if logits_soft_cap < 0:
            raise ValueError("logits_soft_cap must be >= 0")
        self.logits_soft_cap = float(logits_soft_cap)
        self.num_queries_per_kv = self.num_heads // self.num_kv_heads
        support_head_sizes = MetaAttentionBackend.get_supported_head_sizes()
        if self.head_size not in support_head_sizes:
            raise ValueError(f"Head size {head_size} is not supported by MetaAttention. "
                             f"Supported head sizes are {support_head_sizes}.")
        if self.head_size != 128 and self.kv_cache_dtype.startswith("fp8"):
            raise NotImplementedError(f"MetaAttention: the fp8 kv-cache kernels are built for head size 128, not {head_size}")
        self.attn_type = attn_type

    def forward(
        self,
        layer,
        query: torch.Tensor,
        key: torch.Tensor,
        value: torch.Tensor,
        query2: Optional[torch.Tensor],
        key2: Optional[torch.Tensor],
        value2: Optional[torch.Tensor],
        kv_cache: torch.Tensor,
        attn_metadata: MetaAttentionMetadata,
        output: Optional[torch.Tensor] = None,
        output_scale: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """query [T, Hq, D]; key/value [T, Hkv, D]; kv_cache [2, nb, bs, Hkv, D] (numel 0 for the
        profiling run); `output` [T, Hq, D] is written in place and returned (:703-982)."""
        assert output is not None, "Output tensor must be provided."
        if output_scale is not None:
            raise NotImplementedError("fused output quantization is not supported in MetaAttention.")
        fp8_kv = self.kv_cache_dtype.startswith("fp8")
        k_scale_f, v_scale_f = float(getattr(layer, "_k_scale_float", 1.0)), float(getattr(layer, "_v_scale_float", 1.0))
        assert fp8_kv or (k_scale_f == 1.0 and v_scale_f == 1.0), (
            "key/v_scale is only supported with an fp8 kv-cache")
        attn_type = self.attn_type
        if attn_type == AttentionType.ENCODER and not attn_metadata.is_all_encoder_attn_metadata_set:
            raise AttributeError("Encoder attention requires setting encoder metadata attributes.")
        if attn_type == AttentionType.ENCODER_DECODER and not attn_metadata.is_all_cross_attn_metadata_set:
            raise AttributeError("Encoder/decoder cross-attention requires setting cross-attention "
                                 "metadata attributes.")
        if attn_type != AttentionType.DECODER:
            raise NotImplementedError("only decoder self-attention is built on the gfx950 path")
        # Meta tokens (:817-819, fa_kernel_metatoken.py:124-280): every query also attends, without a
        # mask, to num_meta_tokens cached rows key2/value2 shared by all sequences; in a prompt step
        # the meta tokens' own queries (query2) attend to those rows only and their outputs come
        # first in `output`.
        with_meta = key2 is not None or value2 is not None
        if query2 is not None and not with_meta:
            raise ValueError("query2 needs key2 and value2")
        if with_meta:
            if key2 is None or value2 is None:
                raise ValueError("key2 and value2 go together")
            key2 = key2.view(-1, self.num_kv_heads, self.head_size)
            value2 = value2.view(-1, self.num_kv_heads, self.head_size)
            if key2.shape[0] != self.num_meta_tokens or value2.shape != key2.shape:
                raise AssertionError(f"key2/value2 must hold num_meta_tokens = {self.num_meta_tokens} rows")

        window_left = self.sliding_window[0]
        query = query.view(-1, self.num_heads, self.head_size)
        output = output.view(-1, self.num_heads, self.head_size)
        if key is not None:
            key = key.view(-1, self.num_kv_heads, self.head_size)
            value = value.view(-1, self.num_kv_heads, self.head_size)

        # A pure decode step (one new token per sequence, the hot loop) appends and attends in ONE
        # launch: the attention kernel takes the newest K/V row from `key`/`value` and stores it at
        # its slot. Every other step appends first, exactly as the reference does (:790-799).
        int8_kv = isinstance(kv_cache, Int8KVCache)
        scales = dict(k_scale=kv_cache.scales[0], v_scale=kv_cache.scales[1]) if int8_kv else {}
        if fp8_kv:
            if int8_kv:
                raise ValueError("kv_cache_dtype says fp8 but the cache is an Int8KVCache")
            scales = dict(fp8_scales=(k_scale_f, v_scale_f))
            # queries take the fp8 round trip as well (scaled_fp8_quant with layer._q_scale, :806-811)
            query = ops.fp8_round(query.contiguous(), float(getattr(layer, "_q_scale_float", 1.0)))
        byte_kv = int8_kv or fp8_kv
        fuse_append = (kv_cache.numel() > 0 and key is not None and value is not None and not byte_kv
                       and attn_metadata.num_prefill_tokens == 0 and attn_metadata.num_decode_tokens > 0
                       and (attn_metadata.max_decode_query_len or 1) == 1
                       and query.dtype in (torch.bfloat16, torch.float16)
                       and attn_metadata.slot_mapping is not None)
        if kv_cache.numel() > 0:
            key_cache, value_cache = (kv_cache.codes[0], kv_cache.codes[1]) if int8_kv else (kv_cache[0], kv_cache[1])
            if fp8_kv and key_cache.dtype not in (torch.uint8, torch.float8_e4m3fn):
                raise ValueError(f"an fp8 kv-cache must be a uint8 or float8_e4m3fn tensor, got {key_cache.dtype}")
            if key is not None and value is not None and fp8_kv:
                ops.kv_append_fp8(key, value, key_cache, value_cache, attn_metadata.slot_mapping.flatten(),
                                  k_scale_f, v_scale_f)
            elif key is not None and value is not None and int8_kv:
                # rows are quantised on their way in: 128 code bytes + one scale per (token, kv head)
                ops.kv_append_int8(key, value, key_cache, value_cache, scales["k_scale"], scales["v_scale"],
                                   attn_metadata.slot_mapping.flatten())
            elif key is not None and value is not None and not fuse_append:
                # all new K/V of the step (prefill and decode tokens) go in with one launch (:790-799)
                ops.kv_append(key, value, key_cache, value_cache, attn_metadata.slot_mapping.flatten())

        num_prefill_query_tokens = attn_metadata.num_prefill_tokens
        num_decode_query_tokens = attn_metadata.num_decode_tokens
        num_meta_prefill_tokens = num_prefill_query_tokens
        if query2 is not None:
            query2 = query2.view(-1, self.num_heads, self.head_size)
            if query2.shape[0] != self.num_meta_tokens:
                raise AssertionError(f"query2 must hold num_meta_tokens = {self.num_meta_tokens} rows")
            num_meta_prefill_tokens += self.num_meta_tokens
            options = {}
            if self.logits_soft_cap > 0 or self.alibi_slopes is not None:
                # the meta tokens' own queries are the last rows of the prompt call's stacked second attention
                # (fa_kernel_metatoken.py:258-275: q = cat(q1, q2))
                if self.alibi_slopes is not None and self.alibi_slopes.device != query.device:
                    self.alibi_slopes = self.alibi_slopes.to(query.device)
                options = dict(softcap=self.logits_soft_cap, alibi_slopes=self.alibi_slopes,
                               meta_bias=(num_prefill_query_tokens, num_prefill_query_tokens + self.num_meta_tokens))
            output[:self.num_meta_tokens] = ops.meta_token_attention(query2, key2, value2, self.scale, **options)[0]
        prefill_output = output[num_meta_prefill_tokens - num_prefill_query_tokens:num_meta_prefill_tokens]
        decode_output = output[num_meta_prefill_tokens:]

        # The kernels take the meta rows into their own softmax (meta_k/meta_v), over element and byte-code
        # caches alike (the reference runs a second attention over them and merges by log-sum-exp).
        meta_kv = dict(meta_k=key2, meta_v=value2) if with_meta else {}
        # The two score options (:758-759, handed to every flash-attn call of the step) travel with the
        # meta rows' arguments to whichever kernel takes a piece of the step.
        prefill_kv, decode_kv = meta_kv, meta_kv
        if self.logits_soft_cap > 0 or self.alibi_slopes is not None:
            if self.alibi_slopes is not None and self.alibi_slopes.device != query.device:
                self.alibi_slopes = self.alibi_slopes.to(query.device)
            options = dict(softcap=self.logits_soft_cap, alibi_slopes=self.alibi_slopes)
            # the meta rows' ALiBi term follows the reference's second attention call, which stacks the queries of
            # the prompt call (prompt tokens, then the meta tokens' own queries) resp. of the decode call into
            # one sequence (fa_kernel_metatoken.py:169-188, 258-275)
            prefill_kv = dict(meta_kv, **options)
            decode_kv = dict(meta_kv, **options)
            if with_meta:
                prefill_kv["meta_bias"] = (0, num_meta_prefill_tokens)
                decode_kv["meta_bias"] = (0, num_decode_query_tokens)

        decode_query = query[num_prefill_query_tokens:]
        query = query[:num_prefill_query_tokens]
        assert query.shape[0] == num_prefill_query_tokens
        assert decode_query.shape[0] == num_decode_query_tokens

        if prefill_meta := attn_metadata.prefill_metadata:
            if kv_cache.numel() == 0 or prefill_meta.block_tables is None or prefill_meta.block_tables.numel() == 0:
                # plain prompt run: keys and values are the in-flight tensors (:835-884)
                pk, pv = key[:num_prefill_query_tokens], value[:num_prefill_query_tokens]
                if int8_kv:   # attend to what the cache will hold: the rows as quantize_sym returns them
                    pk, pv = ops.quantize_sym(pk), ops.quantize_sym(pv)
                elif fp8_kv:  # scaled_fp8_quant of the prompt's keys and values (:853-869)
                    pk, pv = ops.fp8_round(pk.contiguous(), k_scale_f), ops.fp8_round(pv.contiguous(), v_scale_f)
                self._varlen_inflight(query, pk, pv, prefill_meta, prefill_output, window_left, meta_kv=prefill_kv)
            else:
                # prefix hit / chunked prefill: keys and values come from the paged cache (:885-919)
                assert prefill_meta.seq_lens is not None
                assert prefill_meta.query_start_loc is not None
                self._varlen_paged(query, key_cache, value_cache, prefill_meta.query_start_loc,
                                   prefill_meta.seq_lens_tensor, prefill_meta.block_tables,
                                   max(prefill_meta.seq_lens), prefill_output, window_left,
                                   meta=prefill_meta, scales=scales, meta_kv=prefill_kv)
        if decode_meta := attn_metadata.decode_metadata:
            assert decode_meta.max_decode_query_len is not None
            if decode_meta.max_decode_query_len > 1:
                # several query tokens per decoding sequence (:924-953)
                assert decode_meta.query_start_loc is not None
                self._varlen_paged(decode_query, key_cache, value_cache, decode_meta.query_start_loc,
                                   decode_meta.seq_lens_tensor, decode_meta.block_tables,
                                   decode_meta.max_decode_seq_len, decode_output, window_left,
                                   meta=decode_meta, scales=scales, meta_kv=decode_kv)
            else:
                # one query token per sequence (:954-981); K/V were appended above, or are appended
                # by this very launch when the step is a pure decode step
                n = decode_query.shape[0]
                fused = {}
                if fuse_append:
                    fused = dict(new_key=key[:n], new_value=value[:n],
                                 new_slot_mapping=decode_meta.slot_mapping.flatten()[:n].contiguous())
                if decode_meta._decode_balanced is None:
                    host_lens = decode_meta.host_seq_lens
                    decode_meta._decode_balanced = bool(
                        host_lens is not None and len(host_lens) >= n and
                        ops.plan_decode_split(n, self.num_kv_heads, decode_meta.max_decode_seq_len or max(host_lens[:n]),
                                              window_left, host_lens[:n]))
                ops.swa_decode_attention(
                    decode_query, key_cache, value_cache, decode_meta.seq_lens_tensor[:n],
                    block_table=decode_meta.block_tables, window_left=window_left, scale=self.scale,
                    out=decode_output, max_seq_len=decode_meta.max_decode_seq_len or None,
                    balanced=False if byte_kv else decode_meta._decode_balanced, **scales, **fused, **decode_kv)
        return output

    # -- multi-query forms: every query token becomes one row of the single-query kernel ----
    @staticmethod
    def _rows(query_start_loc: torch.Tensor, num_tokens: int):
        """(row_seq, index of each token inside its sequence's query run), no host sync."""
        n_seqs = query_start_loc.numel() - 1
        qsl = query_start_loc.to(torch.int64)
        lens = qsl[1:] - qsl[:-1]
        row_seq = torch.repeat_interleave(torch.arange(n_seqs, device=qsl.device), lens, output_size=num_tokens)
        j = torch.arange(num_tokens, device=qsl.device) - qsl[row_seq]
        return row_seq, j, lens

    @staticmethod
    def _plan_for(meta, q):
        """Tile plan for the many-query matrix-core kernel, or None when it cannot take the step
        (fp32, a head size other than 128, host lengths unknown, rows padded beyond the sequences' tokens)."""
        if q.dtype not in (torch.bfloat16, torch.float16) or q.shape[-1] != 128:
            return None
        plan = meta.prefill_plan(q.device)
        if plan is None or plan.total_q != q.shape[0]:
            return None
        return plan

    def _varlen_inflight(self, q, k, v, meta, out, window_left, return_lse=False, meta_kv=None):
        """Returns the fp32 [T, Hq] log-sum-exp when asked for, else None. meta_kv: meta_k/meta_v for the
        kernels to take into their softmax."""
        meta_kv = meta_kv or {}
        T = q.shape[0]
        if T == 0:
            return None
        if k.stride() != v.stride():
            v = v.contiguous()
            k = k.contiguous()
        plan = self._plan_for(meta, q)
        if plan is not None and plan.total_k <= k.shape[0]:
            res = ops.swa_prefill_attention(q, k, v, plan=plan, window_left=window_left, scale=self.scale, out=out,
                                            kv_start=meta.seq_start_loc.to(torch.int64)[:-1].contiguous(),
                                            return_lse=return_lse, **meta_kv)
            return res[1] if return_lse else None
        row_seq, j, _ = self._rows(meta.query_start_loc, T)
        seq_lens_row = (j + 1).to(torch.int32)
        res = ops.swa_decode_attention(
            q, k, v, seq_lens_row, kv_start=meta.seq_start_loc.to(torch.int64)[:-1].contiguous(),
            row_seq=row_seq.to(torch.int32), kv_strides=(0, k.stride(0), k.stride(1)),
            num_kv_heads=self.num_kv_heads, window_left=window_left, scale=self.scale, out=out,
            max_seq_len=meta.max_prefill_seq_len or None, return_lse=return_lse, **meta_kv)
        return res[1] if return_lse else None

    def _varlen_paged(self, q, key_cache, value_cache, query_start_loc, seq_lens_tensor, block_tables,
                      max_seq_len, out, window_left, meta=None, return_lse=False, scales=None, meta_kv=None):
        """scales: k_scale/v_scale of an INT8 cache or fp8_scales of an fp8 cache, passed on to whichever
        kernel takes the step; meta_kv: meta_k/meta_v for that kernel to take into its softmax."""
        meta_kv = meta_kv or {}
        T = q.shape[0]
        if T == 0:
            return None
        scales = scales or {}
        plan = self._plan_for(meta, q) if meta is not None else None
        if plan is not None and block_tables.shape[1] * key_cache.shape[1] >= plan.max_k:
            res = ops.swa_prefill_attention(q, key_cache, value_cache, plan=plan, block_table=block_tables,
                                            window_left=window_left, scale=self.scale, out=out, return_lse=return_lse,
                                            **scales, **meta_kv)
            return res[1] if return_lse else None
        row_seq, j, lens = self._rows(query_start_loc, T)
        # query j of a run of n queries in a sequence of L keys sits at key index L - n + j
        seq_lens_row = (seq_lens_tensor.to(torch.int64)[row_seq] - lens[row_seq] + j + 1).to(torch.int32)
        res = ops.swa_decode_attention(
            q, key_cache, value_cache, seq_lens_row, block_table=block_tables, row_seq=row_seq.to(torch.int32),
            window_left=window_left, scale=self.scale, out=out, max_seq_len=max_seq_len or None,
            return_lse=return_lse, **scales, **meta_kv)
        return res[1] if return_lse else None
