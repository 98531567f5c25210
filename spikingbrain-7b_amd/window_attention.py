"""Cache + attention slice of the HuggingFace-side sliding-window layer.

Mirrors the part of `FlashAttention.forward` between RoPE and `o_proj`:
  hf_7B_model/window_attention.py:164-217      (flash flavour: window_size=(W, 0), i.e. the query
                                                sees itself and W keys to its left)
  hf_7B_model/window_attention_sdpa.py:174-214 (SDPA flavour: W keys including itself, and no
                                                window_size handed to the cache, :176)
Projections, RoPE and o_proj stay with the caller; inputs are the post-RoPE q/k/v.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops
from .hf_cache import Cache


# query runs at least this long use the many-query kernel; shorter ones (speculative / multi-token
# decode) run as rows of the single-query kernel, which wastes no tile rows on them
PREFILL_MIN_QUERIES = 16

_plans: dict = {}


def _uniform_plan(B: int, Q: int, K: int, dev: torch.device):
    """Tile plan for B sequences of Q queries over K keys each (every layer of a forward pass asks
    for the same one)."""
    key = (B, Q, K, dev)
    plan = _plans.get(key)
    if plan is None:
        if len(_plans) >= 64:
            _plans.clear()
        plan = _plans[key] = ops.PrefillPlan([Q] * B, [K] * B, dev)
    return plan


def _kv_start_rows(k: torch.Tensor) -> Optional[torch.Tensor]:
    """Row offset of each batch entry, in units of k.stride(2); None if it is not a whole number."""
    B = k.shape[0]
    if B == 1:
        return torch.zeros(1, dtype=torch.int64, device=k.device)
    if k.stride(2) == 0 or k.stride(0) % k.stride(2) != 0:
        return None
    return torch.arange(B, dtype=torch.int64, device=k.device) * (k.stride(0) // k.stride(2))


def sliding_window_attention(
    query_states: torch.Tensor,
    key_states: torch.Tensor,
    value_states: torch.Tensor,
    sliding_window: int,
    past_key_values: Optional[Cache] = None,
    layer_idx: int = 0,
    attention_mask: Optional[torch.Tensor] = None,
    flavour: str = "flash",
    cache_window_size: Optional[int] = -1,
    window_left: Optional[int] = None,
) -> torch.Tensor:
    """query_states [B, Hq, Q, D]; key_states/value_states [B, Hkv, Q, D] (new tokens only).
    Appends the new K/V to `past_key_values` exactly as the reference layer does, then attends
    causally inside the sliding window over the cached (or, on the first call, the in-flight)
    keys. `attention_mask` [B, >=K] marks left padding with 0. Returns [B, Q, Hq, D].
    `flavour` picks the two conventions the reference files use (flash: cache bounded at W rows,
    W keys left of the query visible; sdpa: cache unbounded, W keys including the query);
    `cache_window_size` (None = unbounded) and `window_left` override them one by one, e.g. a
    bounded cache with the SDPA mask.
    A fully masked query row (a pad position) comes out as zeros."""
    if flavour not in ("flash", "sdpa"):
        raise ValueError("flavour must be 'flash' or 'sdpa'")
    B, Hq, Q, D = query_states.shape
    Hkv = key_states.shape[1]

    if past_key_values is not None:
        cache_has_content = past_key_values.get_seq_length(layer_idx) > 0
        if cache_window_size == -1:
            cache_kwargs = {"window_size": sliding_window} if flavour == "flash" else {}
        else:
            cache_kwargs = {"window_size": cache_window_size}
        key_cached, value_cached = past_key_values.update(
            attn_state=(key_states, value_states), layer_idx=layer_idx, offset=Q,
            cache_kwargs=cache_kwargs)["attn_state"]
        if cache_has_content:
            key_states, value_states = key_cached, value_cached

    K = key_states.shape[2]
    if window_left is None:
        window_left = sliding_window if flavour == "flash" else sliding_window - 1

    k, v = key_states, value_states
    if k.stride(3) != 1 or v.stride() != k.stride() or _kv_start_rows(k) is None:
        k, v = k.contiguous(), v.contiguous()
    kv_start = _kv_start_rows(k)

    q_rows = query_states.transpose(1, 2).reshape(B * Q, Hq, D)
    dev = q_rows.device
    if Q >= PREFILL_MIN_QUERIES and q_rows.dtype in (torch.bfloat16, torch.float16) and D == 128:
        # prompt-sized query runs go to the matrix-core kernel (64-token tiles)
        pad = None
        if attention_mask is not None:
            pad = (K - (attention_mask[:, -K:] != 0).sum(dim=1)).to(torch.int32).contiguous()
        out = ops.swa_prefill_attention(
            q_rows, k, v, plan=_uniform_plan(B, Q, K, dev), kv_start=kv_start, key_lo=pad,
            kv_strides=(k.stride(2), k.stride(1)), num_kv_heads=Hkv, window_left=window_left, scale=D ** -0.5)
        return out.view(B, Q, Hq, D)
    j = torch.arange(Q, device=dev, dtype=torch.int32)
    seq_lens_row = (K - Q + 1 + j).repeat(B)                       # query j sits at key index K - Q + j
    row_seq = torch.arange(B, device=dev, dtype=torch.int32).repeat_interleave(Q)
    key_lo = None
    if attention_mask is not None:
        keep = attention_mask[:, -K:]
        pad = (K - (keep != 0).sum(dim=1)).to(torch.int32)         # left padding: zeros form a prefix
        key_lo = pad.repeat_interleave(Q)
    out = ops.swa_decode_attention(
        q_rows, k, v, seq_lens_row, kv_start=kv_start, row_seq=row_seq, key_lo=key_lo,
        kv_strides=(0, k.stride(2), k.stride(1)), num_kv_heads=Hkv, window_left=window_left,
        scale=D ** -0.5, max_seq_len=K)
    return out.view(B, Q, Hq, D)
