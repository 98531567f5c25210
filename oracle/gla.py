"""numpy (float64) restatement of the GLA recurrent step on the path.

TEST INFRASTRUCTURE: see oracle/__init__.py.
"""
from __future__ import annotations

from typing import Optional

import numpy as np


def gla_step(q, k, v, g, state, slot_idx=None, scale: Optional[float] = None):
    """vllm_hymeta/model_for_7B/my_fused_recurrent.py:27-80 (launcher :88-119, wrapper :138-153).

    q, k, v, g: [B, H, D] (the reference passes [B, H, 1, D]); state: [slots, H, dk, dv], updated IN
    PLACE; slot_idx: [B] ints, -1 = row skipped (nothing read or written, :32-36).
        q_s   = q * scale                          (:60, scale default D^-0.5 :96-97)
        S_new = k[:, None] * v[None, :] + exp(g)[:, None] * S_old      (:65-72)
        o     = sum_dk q_s[:, None] * S_new        (:75-76, the UPDATED state)
    Returns o [B, H, D] float64; rows with slot -1 are NaN (the reference leaves them
    uninitialised)."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    g = np.asarray(g, np.float64)
    B, H, D = q.shape
    if scale is None:
        scale = D ** -0.5
    o = np.full((B, H, D), np.nan)
    for b in range(B):
        slot = b if slot_idx is None else int(slot_idx[b])
        if slot == -1:
            continue
        for h in range(H):
            S = np.asarray(state[slot, h], np.float64)
            S_new = k[b, h][:, None] * v[b, h][None, :] + np.exp(g[b, h])[:, None] * S
            o[b, h] = ((q[b, h] * scale)[:, None] * S_new).sum(0)
            state[slot, h] = S_new
    return o


def gla_recurrent(q, k, v, g, initial_state=None, scale: Optional[float] = None):
    """T-step form: fla.ops.gla.fused_recurrent_gla as called at hf_7B_model/gla_attention.py:153
    (recurrence of the technical report, eq. (10)-(11)); q, k, v, g [B, H, T, D] head-first.
    Returns (o [B, H, T, D], final_state [B, H, D, D]) float64."""
    q = np.asarray(q, np.float64)
    B, H, T, D = q.shape
    S = np.zeros((B, H, D, D)) if initial_state is None else np.array(initial_state, np.float64)
    o = np.zeros((B, H, T, D))
    for t in range(T):
        o[:, :, t] = gla_step(q[:, :, t], np.asarray(k)[:, :, t], np.asarray(v)[:, :, t],
                              np.asarray(g)[:, :, t], S.reshape(B, H, D, D), None, scale)
    return o, S
