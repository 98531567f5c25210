"""GLA recurrent-state path: the kernel entry points the reference's GLA layers call, and the
constant-size slot cache that holds the per-layer states.

Mirrors
  vllm_hymeta/model_for_7B/my_fused_recurrent.py:138-153   my_fused_recurrent_gla
  hf_7B_model/gla_attention.py:153                         fused_recurrent_gla (fla, un-vendored)
  vllm_hymeta/model_for_7B/gla_cache.py:7-32               GLACacheParams, GLACacheManager
  vllm_hymeta/model_for_7B/modeling_gla_swa.py:391-414     slot clearing for new prefills
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Iterable, List, Optional, Tuple

import torch

from . import ops

PAD_SLOT_ID = -1


def my_fused_recurrent_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor = None,
    kv_caches: torch.Tensor = None,
    slot_idx: torch.Tensor = None,
    scale: Optional[float] = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    reverse: bool = False,
) -> torch.Tensor:
    """Single-token GLA decode with the state cache updated in place.

    q, k, v, g: [B, H, 1, D]; kv_caches: [slots, H, D, D]; slot_idx: [B] int (-1 = skip the row).
    Returns o [B, H, D] (my_fused_recurrent.py:117-119). `initial_state`, `output_final_state`
    and `reverse` are accepted and ignored, as in the reference (:88-119 never reads them).
    Rows whose slot is -1 keep whatever the output buffer held (the reference leaves them
    uninitialised); here the buffer starts zeroed.

    Shared states (not in the reference, which repeats k, v and the gate to all query heads before this
    call, gla_attention.py:264-267): k, v, g [B, Hkv, 1, D] and kv_caches [slots, Hkv, D, D] with H a
    multiple of Hkv give the same outputs from one state per kv head."""
    if q.dim() != 4 or q.shape[2] != 1:
        raise AssertionError(f"decode expects q of shape [B, H, 1, D], got {tuple(q.shape)}")
    B, H, _, D = q.shape
    assert k.dim() == 4 and (k.shape[0], k.shape[2], k.shape[3]) == (B, 1, D) and H % k.shape[1] == 0
    assert v.shape == k.shape
    if scale is None:
        scale = D ** -0.5
    if slot_idx is not None and slot_idx.dtype != torch.int32:
        slot_idx = slot_idx.to(torch.int32)
    out = torch.zeros((B, H, 1, D), dtype=q.dtype, device=q.device)
    ops.gla_recurrent(q, k, v, g, kv_caches, slot_idx, scale, out)
    return out.view(B, H, D)


def fused_recurrent_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    gk: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    inplace_state: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """T-step recurrence on head-first tensors [B, H, T, D], the call made at
    hf_7B_model/gla_attention.py:153: returns (o [B, H, T, D], final_state [B, H, D, D] fp32 or None).
    The state crosses HBM once in each direction whatever T is. With inplace_state=True an fp32
    `initial_state` is advanced in place and returned (the cache replaces it by reference anyway,
    hf_7B_model/cache.py:92-93), saving the copy. With k, v, gk of Hkv < H heads the state is
    [B, Hkv, D, D], shared by each group of H / Hkv query heads."""
    B, H, T, D = q.shape
    if initial_state is None:
        state = torch.zeros((B, k.shape[1], D, D), dtype=torch.float32, device=q.device)
    elif inplace_state and initial_state.dtype == torch.float32 and initial_state.is_contiguous():
        state = initial_state
    else:
        state = initial_state.to(torch.float32, copy=True).contiguous()
    o = ops.gla_recurrent(q, k, v, gk, state, None, scale)
    return o, (state if output_final_state else None)


def fused_chunk_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    scale: float = -1,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Name and call shape of fla's chunked GLA kernel as the reference's prefill loop uses it
    (vllm_hymeta/model_for_7B/gla_attention.py:207-208): q, k, v, g [B, H, T, D], returns
    (o [B, H, T, D], final_state [B, H, D, D] fp32 or None). Computed by the many-step recurrent
    kernel (same mathematics, state crossing HBM once); scale -1 means D^-0.5 as in fla."""
    return fused_recurrent_gla(q, k, v, g, None if scale == -1 else scale, initial_state, output_final_state)


def gla_prefill_packed(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gk: torch.Tensor, kv_cache: torch.Tensor,
                       state_indices_tensor: torch.Tensor, query_start_loc: torch.Tensor, num_prefills: int,
                       max_query_len: Optional[int] = None) -> torch.Tensor:
    """The prefill half of `_prefill_and_mix_infer` (vllm_hymeta/model_for_7B/gla_attention.py:179-214)
    as ONE launch: q, k, v, gk [num_tokens, H, D] with the prefill tokens first; prompt i owns tokens
    query_start_loc[i] .. query_start_loc[i+1]-1, starts from the state in kv_cache[slot_i] (the
    runner zeroes the slots of new prompts, `clear_prefill_slots`) and leaves its final state there,
    with no per-request Python loop, slice copies or state copy. Returns o for the prefill tokens
    [num_prefill_tokens, H, D] (before g_norm)."""
    n = int(num_prefills)
    cu = query_start_loc[:n + 1].to(torch.int32).contiguous()
    slots = state_indices_tensor[:n].to(torch.int32).contiguous()
    return ops.gla_recurrent_packed(q, k, v, gk, kv_cache, cu, slots, max_seq_len=max_query_len)


@dataclass
class GLACacheParams:
    """gla_cache.py:7-14."""
    gla_cache: torch.Tensor = field(default_factory=torch.Tensor)
    state_indices_tensor: torch.Tensor = field(default_factory=torch.Tensor)

    def at_layer_idx(self, layer_idx: int) -> "GLACacheParams":
        return GLACacheParams(self.gla_cache[layer_idx, ...], self.state_indices_tensor)


class ConstantSizeCache:
    """Request -> slot bookkeeping of a cache with one fixed-size entry per running sequence
    (the role vLLM's `ConstantSizeCache` base class plays for gla_cache.py:16): free slots form a
    stack that pops the highest index first; finished requests give their slots back; a new
    sequence of a known request (parallel sampling) gets a copy of a sibling's entry."""

    def __init__(self, max_batch_size: int):
        self.cache_indices_mapping: Dict[str, Dict[int, int]] = {}
        self.free_cache_indices: List[int] = list(range(max_batch_size))

    @property
    def cache(self):
        raise NotImplementedError

    def _copy_cache(self, from_index: int, to_index: int) -> None:
        raise NotImplementedError

    def _release_finished_requests(self, finished_requests_ids: Iterable[str]) -> None:
        for req_id in finished_requests_ids:
            slots = self.cache_indices_mapping.pop(req_id, None)
            if slots:
                self.free_cache_indices.extend(slots.values())

    def _slot_for(self, req_id: str, seq_id: int, finished_requests_ids) -> int:
        if req_id in finished_requests_ids:
            return PAD_SLOT_ID
        known = self.cache_indices_mapping.get(req_id)
        if known is None:
            slot = self.free_cache_indices.pop()
            self.cache_indices_mapping[req_id] = {seq_id: slot}
            return slot
        if seq_id not in known:
            source = next(iter(known.values()))
            slot = self.free_cache_indices.pop()
            self._copy_cache(from_index=source, to_index=slot)
            known[seq_id] = slot
            return slot
        return known[seq_id]

    def _prepare_current_run_cache(self, request_ids_to_seq_ids: Dict[str, List[int]],
                                   finished_requests_ids: List[str]) -> List[int]:
        return [self._slot_for(req_id, seq_id, finished_requests_ids)
                for req_id, seq_ids in request_ids_to_seq_ids.items() for seq_id in seq_ids]

    def current_run_tensors(self, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
        """(cache tensor, state_indices int32 [num_seqs]) for this engine step; call as the model
        does at vllm_hymeta/model_for_7B/modeling_gla_swa.py:444-447."""
        if "seqlen_agnostic_capture_inputs" in kwargs:
            return kwargs["seqlen_agnostic_capture_inputs"]
        finished = kwargs["finished_requests_ids"]
        self._release_finished_requests(finished)
        indices = self._prepare_current_run_cache(kwargs["request_ids_to_seq_ids"], finished)
        return self.cache, torch.as_tensor(indices, dtype=torch.int32, device=self.cache.device)

    def copy_inputs_before_cuda_graphs(self, input_buffers, **kwargs) -> None:
        finished = kwargs["finished_requests_ids"]
        self._release_finished_requests(finished)
        indices = self._prepare_current_run_cache(kwargs["request_ids_to_seq_ids"], finished)
        _, buf = input_buffers["seqlen_agnostic_capture_inputs"]
        indices.extend([PAD_SLOT_ID] * (buf.shape[0] - len(indices)))
        buf.copy_(torch.as_tensor(indices, dtype=torch.int32), non_blocking=True)

    def get_seqlen_agnostic_capture_inputs(self, batch_size: int):
        return self.cache, torch.full((batch_size,), PAD_SLOT_ID, dtype=torch.int32, device=self.cache.device)


class GLACacheManager(ConstantSizeCache):
    """gla_cache.py:16-32: one tensor [n_gla_layers, max_num_seqs, H, D, D] holding every GLA
    layer's state for every slot (shape built at modeling_gla_swa.py:348-356)."""

    def __init__(self, dtype: torch.dtype, cache_shape: Tuple[int, ...], device="cuda"):
        super().__init__(cache_shape[1])
        # uninitialised, like the reference; slots are zeroed when a new prefill claims them
        self._gla_cache = torch.empty(size=cache_shape, dtype=dtype, device=device)

    @property
    def cache(self) -> torch.Tensor:
        return self._gla_cache

    def _copy_cache(self, from_index: int, to_index: int) -> None:
        # Copies the slot in every layer. (The reference loops over layers and then indexes
        # dim 1 of the per-layer view, which is the head axis, gla_cache.py:28-32; the intent,
        # a sibling copy of the whole slot, is what is done here.)
        self._gla_cache[:, to_index].copy_(self._gla_cache[:, from_index], non_blocking=True)

    def clear_slots(self, slots: List[int]) -> None:
        """Zero the given slots in all layers (modeling_gla_swa.py:406-414)."""
        if slots:
            idx = torch.tensor(slots, device=self._gla_cache.device, dtype=torch.long)
            self._gla_cache[:, idx, ...] = 0


def clear_prefill_slots(manager: GLACacheManager, num_prefills: int, context_lens: List[int],
                        request_ids_to_seq_ids: Dict[str, List[int]]) -> List[int]:
    """Slots of brand-new prompts (context_len == 0) are zeroed before the layers run
    (modeling_gla_swa.py:391-414). `context_lens` is a host list (one entry per prefill)."""
    seq_to_slot: Dict[int, int] = {}
    for m in manager.cache_indices_mapping.values():
        seq_to_slot.update(m)
    seq_ids = [s for ids in request_ids_to_seq_ids.values() for s in ids]
    slots = [seq_to_slot[seq_ids[i]] for i in range(min(num_prefills, len(seq_ids)))
             if context_lens[i] == 0 and seq_ids[i] in seq_to_slot]
    manager.clear_slots(slots)
    return slots
