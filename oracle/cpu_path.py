"""The reference's PyTorch CPU path for one decode step, restated with plain torch CPU ops.

TEST INFRASTRUCTURE (see oracle/__init__.py): this is what `bench.py` times as `cpu_baseline`
(kind "port"); the parity tests use the numpy oracles (hf_cache, attention, gla) instead. Pinned by
tests/test_oracle_cpu_path.py: the window update against an independent list-of-rows model (the
300/511/700/900 traces at W=512, random schedules, the overshoot quirk), the attention against a
mask-and-softmax loop written from the prose (left padding, fully masked queries), the GLA step
against the float64 unrolled closed form and its special cases. It follows
  - hf_7B_model/cache.py:94-107        dense sliding-window update (roll + slice-assign / cat)
  - hf_7B_model/window_attention_sdpa.py:82-91,140-148,186-214   repeat_kv + SDPA with the
                                       sliding-causal additive mask + nan_to_num
  - vllm_hymeta/model_for_7B/my_fused_recurrent.py:60-80         GLA single-token update
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def dense_window_update(key_state: Optional[torch.Tensor], value_state: Optional[torch.Tensor],
                        k_new: torch.Tensor, v_new: torch.Tensor, window_size: Optional[int]
                        ) -> Tuple[torch.Tensor, torch.Tensor]:
    """cache.py:79-89 (first call) and :94-107 (later calls) for one layer's (K, V) pair."""
    n = k_new.shape[-2]
    if key_state is None:
        if window_size is not None and n > window_size:
            return k_new[..., -window_size:, :].contiguous(), v_new[..., -window_size:, :].contiguous()
        return k_new, v_new
    if window_size is not None and key_state.shape[-2] == window_size:
        key_state = key_state.roll(-n, -2)
        value_state = value_state.roll(-n, -2)
        key_state[..., -n:, :] = k_new
        value_state[..., -n:, :] = v_new
        return key_state, value_state
    return torch.cat([key_state, k_new], -2), torch.cat([value_state, v_new], -2)


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """window_attention_sdpa.py:82-91."""
    b, h, l, d = x.shape
    if n_rep == 1:
        return x
    return x[:, :, None, :, :].expand(b, h, n_rep, l, d).reshape(b, h * n_rep, l, d)


def sdpa_window_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sliding_window: int,
                          attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """window_attention_sdpa.py:186-214 on q [B,Hq,Q,D], k/v [B,Hkv,K,D]."""
    B, Hq, Q, D = q.shape
    K = k.shape[2]
    k = repeat_kv(k, Hq // k.shape[1])
    v = repeat_kv(v, Hq // v.shape[1])
    k_pos = torch.arange(K)
    q_abs = (K - Q) + torch.arange(Q)
    allowed = (k_pos[None, :] <= q_abs[:, None]) & (k_pos[None, :] > (q_abs[:, None] - sliding_window))
    mask = (~allowed).view(1, 1, Q, K)
    if attention_mask is not None:
        mask = mask | (attention_mask[:, -K:] == 0).view(B, 1, 1, K)
    add = torch.where(mask, -torch.inf, 0.0).to(q.dtype)
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=add, dropout_p=0.0, is_causal=False)
    return torch.nan_to_num(out, nan=0.0)


def gla_step(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
             scale: Optional[float] = None) -> torch.Tensor:
    """my_fused_recurrent.py:60-80 with identity slots, fp32 math, state [B,H,dk,dv] in place."""
    if scale is None:
        scale = q.shape[-1] ** -0.5
    state.mul_(g.float().exp().unsqueeze(-1)).add_(k.float().unsqueeze(-1) * v.float().unsqueeze(-2))
    return torch.einsum("bhk,bhkv->bhv", q.float() * scale, state)
