"""numpy restatement of the sliding-window attention math on the path.

TEST INFRASTRUCTURE: see oracle/__init__.py. float64 throughout unless a dtype is given.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import numpy as np


def repeat_kv(x: np.ndarray, n_rep: int) -> np.ndarray:
    """hf_7B_model/window_attention.py:82-91: [B, Hkv, L, D] -> [B, Hkv*n_rep, L, D], each kv head
    repeated n_rep times consecutively (query head hq reads kv head hq // n_rep)."""
    if n_rep == 1:
        return x
    b, h, l, d = x.shape
    return np.broadcast_to(x[:, :, None], (b, h, n_rep, l, d)).reshape(b, h * n_rep, l, d)


def sliding_causal_mask(q_len: int, k_len: int, window_size: int) -> np.ndarray:
    """hf_7B_model/window_attention_sdpa.py:140-148. True = masked.
    Key k is visible to query i iff k <= q_abs and k > q_abs - window_size, q_abs = (K-Q)+i,
    i.e. window_size keys including the query's own position."""
    k_pos = np.arange(k_len)
    q_abs = (k_len - q_len) + np.arange(q_len)
    allowed = (k_pos[None, :] <= q_abs[:, None]) & (k_pos[None, :] > (q_abs[:, None] - window_size))
    return ~allowed


def masked_softmax_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, masked: np.ndarray,
                             scale: Optional[float] = None, return_lse: bool = False,
                             softcap: float = 0.0, bias: Optional[np.ndarray] = None):
    """softmax(q k^T * scale + (-inf where masked)) v with fully-masked rows -> 0
    (window_attention_sdpa.py:205-214: additive -inf mask, SDPA default scale D^-0.5,
    nan_to_num(nan=0)). q [..., Q, D], k/v [..., K, D], masked broadcastable to [..., Q, K].
    softcap > 0 and bias are the two options the backend hands to flash-attn
    (vllm_hymeta/attention/meta_attention.py:686-690 logits_soft_cap, :665-670 alibi_slopes;
    fa_kernel_metatoken.py:157-168, 235-253 pass them on as softcap / alibi_slopes): the scaled
    scores become softcap * tanh(scores / softcap), then the bias (broadcastable to [..., Q, K]) is
    added, then the mask."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    if scale is None:
        scale = q.shape[-1] ** -0.5
    s = np.einsum("...qd,...kd->...qk", q, k) * scale
    if softcap > 0:
        s = softcap * np.tanh(s / softcap)
    if bias is not None:
        s = s + np.asarray(bias, np.float64)
    s = np.where(masked, -np.inf, s)
    mx = s.max(axis=-1, keepdims=True)
    mx_safe = np.where(np.isfinite(mx), mx, 0.0)
    p = np.exp(s - mx_safe)
    l = p.sum(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        out = np.where(l > 0, np.einsum("...qk,...kd->...qd", p, v) / np.where(l > 0, l, 1.0), 0.0)
        lse = np.where(l[..., 0] > 0, np.log(np.where(l[..., 0] > 0, l[..., 0], 1.0)) + mx_safe[..., 0], -np.inf)
    return (out, lse) if return_lse else out


def sdpa_window_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, sliding_window: int,
                          attention_mask: Optional[np.ndarray] = None) -> np.ndarray:
    """The attention slice of hf_7B_model/window_attention_sdpa.py:186-214.
    q [B, Hq, Q, D]; k, v [B, Hkv, K, D] (un-repeated); attention_mask [B, >=K] with 0 = pad.
    Returns [B, Hq, Q, D] float64."""
    B, Hq, Q, D = q.shape
    Hkv, K = k.shape[1], k.shape[2]
    kr = repeat_kv(np.asarray(k, np.float64), Hq // Hkv)
    vr = repeat_kv(np.asarray(v, np.float64), Hq // Hkv)
    masked = sliding_causal_mask(Q, K, sliding_window).reshape(1, 1, Q, K)
    if attention_mask is not None:
        key_keep = np.asarray(attention_mask)[:, -K:]  # :198
        pad = (key_keep == 0).reshape(B, 1, 1, K)
        masked = masked | pad
    return masked_softmax_attention(q, kr, vr, masked)


def flash_window_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, sliding_window: int,
                           attention_mask: Optional[np.ndarray] = None) -> np.ndarray:
    """The inference branch of hf_7B_model/window_attention.py:186-217, step by step: the padding mask
    is cut to the key length (attention_mask[:, -K:], :190), pad positions are dropped from K/V and
    from the last Q query positions (_upad_input, :188-193), every sequence runs causal varlen
    attention with window_size = (sliding_window, 0), i.e. the query sees itself and sliding_window
    keys to its left, bottom-right aligned (:204-215), and pad_input puts the rows back with zeros
    at pad positions (:216). q [B, Hq, Q, D]; k, v [B, Hkv, K, D]; returns [B, Hq, Q, D] float64.
    Q is either K (prompt) or 1 (decode), the two cases _upad_input supports with a kv mask."""
    B, Hq, Q, D = q.shape
    K = k.shape[2]
    keep = np.ones((B, K), bool) if attention_mask is None else (np.asarray(attention_mask)[:, -K:] != 0)
    out = np.zeros((B, Hq, Q, D))
    for b in range(B):
        kidx = np.nonzero(keep[b])[0]
        qkeep = keep[b, K - Q:]                    # the queries are the last Q positions
        qidx = np.nonzero(qkeep)[0]
        if len(qidx) == 0:
            continue
        qs = np.asarray(q[b], np.float64)[:, qidx].transpose(1, 0, 2)          # [Lq, Hq, D]
        ks = np.asarray(k[b], np.float64)[:, kidx].transpose(1, 0, 2)          # [Lk, Hkv, D]
        vs = np.asarray(v[b], np.float64)[:, kidx].transpose(1, 0, 2)
        o = varlen_window_attention(qs, ks, vs, [0, len(qidx)], [0, len(kidx)], D ** -0.5, sliding_window)
        out[b][:, qidx] = o.transpose(1, 0, 2)
    return out


def gather_paged(cache: np.ndarray, block_table_row: Sequence[int], n: int) -> np.ndarray:
    """Rows 0..n-1 of a sequence from a paged cache half [num_blocks, bs, Hkv, D] -> [n, Hkv, D]
    (key i lives in block block_table[i // bs] at offset i % bs; kv_cache layout of
    vllm_hymeta/attention/meta_attention.py:81-92)."""
    bs = cache.shape[1]
    nb = (n + bs - 1) // bs
    blocks = np.asarray(block_table_row[:nb], dtype=np.int64)
    return cache[blocks].reshape(nb * bs, cache.shape[2], cache.shape[3])[:n]


def alibi_bias(slope: float, query_pos: np.ndarray, n_keys: int) -> np.ndarray:
    """The ALiBi term flash-attn adds for a query at key position query_pos: -slope * |query_pos - key|
    for every key index (the causal mask removes the keys to the right). Returns [len(query_pos), n_keys]."""
    return -float(slope) * np.abs(np.asarray(query_pos)[:, None] - np.arange(n_keys)[None, :])


def paged_decode_attention(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
                           block_tables: np.ndarray, cache_seqlens: Sequence[int], scale: float,
                           window_left: int, return_lse: bool = False, softcap: float = 0.0,
                           alibi_slopes: Optional[Sequence[float]] = None):
    """Semantics of flash_attn_with_kvcache as called at
    vllm_hymeta/attention/fa_kernel_metatoken.py:157-168: one query per sequence placed at key
    index cache_seqlens-1, causal, window_size=(window_left, -1): key i visible iff
    cache_seqlens-1-window_left <= i <= cache_seqlens-1 (window_left < 0: unbounded).
    q [B, Hq, D]; caches [nb, bs, Hkv, D]; returns [B, Hq, D] float64 (and lse [B, Hq])."""
    B, Hq, D = q.shape
    Hkv = k_cache.shape[2]
    G = Hq // Hkv
    out = np.zeros((B, Hq, D))
    lse = np.full((B, Hq), -np.inf)
    for b in range(B):
        n = int(cache_seqlens[b])
        if n <= 0:
            continue
        kk = gather_paged(k_cache, block_tables[b], n).astype(np.float64)  # [n, Hkv, D]
        vv = gather_paged(v_cache, block_tables[b], n).astype(np.float64)
        i = np.arange(n)
        masked = np.zeros(n, bool) if window_left < 0 else (i < n - 1 - window_left)
        for h in range(Hq):
            bias = None if alibi_slopes is None else alibi_bias(alibi_slopes[h], np.array([n - 1]), n)
            o, ls = masked_softmax_attention(np.asarray(q[b, h], np.float64)[None], kk[:, h // G], vv[:, h // G],
                                             masked[None], scale, return_lse=True, softcap=softcap, bias=bias)
            out[b, h] = o[0]
            lse[b, h] = ls[0]
    return (out, lse) if return_lse else out


def varlen_window_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, cu_seqlens_q: Sequence[int],
                            cu_seqlens_k: Sequence[int], scale: float, window_left: int, softcap: float = 0.0,
                            alibi_slopes: Optional[Sequence[float]] = None) -> np.ndarray:
    """Semantics of the varlen causal sliding-window call at
    vllm_hymeta/attention/fa_kernel_metatoken.py:235-253 (bottom-right aligned causal mask):
    query j of a sequence with Lq queries and Lk keys sits at key position Lk-Lq+j and sees keys
    in [pos-window_left, pos]. q [Tq, Hq, D]; k, v [Tk, Hkv, D]; returns [Tq, Hq, D] float64."""
    Tq, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    out = np.zeros((Tq, Hq, D))
    for s in range(len(cu_seqlens_q) - 1):
        q0, q1 = int(cu_seqlens_q[s]), int(cu_seqlens_q[s + 1])
        k0, k1 = int(cu_seqlens_k[s]), int(cu_seqlens_k[s + 1])
        Lq, Lk = q1 - q0, k1 - k0
        if Lq == 0:
            continue
        pos = (Lk - Lq) + np.arange(Lq)
        kp = np.arange(Lk)
        masked = kp[None, :] > pos[:, None]
        if window_left >= 0:
            masked |= kp[None, :] < (pos[:, None] - window_left)
        for h in range(Hq):
            bias = None if alibi_slopes is None else alibi_bias(alibi_slopes[h], pos, Lk)
            out[q0:q1, h] = masked_softmax_attention(q[q0:q1, h], k[k0:k1, h // G], v[k0:k1, h // G], masked, scale,
                                                     softcap=softcap, bias=bias)
    return out


def lse_merge(out_a: np.ndarray, lse_a: np.ndarray, out_b: np.ndarray, lse_b: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """vllm_hymeta/attention/fa_kernel_metatoken.py:110-122 with out [..., D] and lse [...]:
    new_lse = lse - logsigmoid(lse - lse_b); out = out - sigmoid(lse_b - lse) * (out - out_b)."""
    out_a = np.asarray(out_a, np.float64)
    out_b = np.asarray(out_b, np.float64)
    d = np.asarray(lse_a, np.float64) - np.asarray(lse_b, np.float64)
    logsig = -np.logaddexp(0.0, -d)          # logsigmoid(lse - lse_b)
    sig_rev = 1.0 / (1.0 + np.exp(d))        # sigmoid(lse_b - lse)
    return out_a - sig_rev[..., None] * (out_a - out_b), lse_a - logsig


def metatoken_attention(q1: np.ndarray, q2: Optional[np.ndarray], k1: np.ndarray, k2: np.ndarray,
                        v1: np.ndarray, v2: np.ndarray, scale: float, sliding_window: int,
                        softcap: float = 0.0, alibi_slopes: Optional[Sequence[float]] = None,
                        stack_row0: int = 0, stack_rows: Optional[int] = None) -> np.ndarray:
    """The dense masked-softmax statement of meta-token attention,
    vllm_hymeta/attention/fa_kernel_metatoken.py:372-405, for one sequence: ONE softmax per query
    over [k2 | k1]. Query i of q1 (Lq queries, bottom-right aligned on the Lk keys of k1) sees every
    meta token and the keys k with 0 <= pos_i - k < sliding_window (sliding_window <= 0: no window
    limit); the meta tokens' own queries q2 see the meta tokens only. q1 [Lq, Hq, D], q2 [M, Hq, D]
    or None, k1/v1 [Lk, Hkv, D], k2/v2 [M, Hkv, D]. Returns [Lq (+ M), Hq, D] float64, rows in the
    order (q1, q2) as at :388 (the flash path moves the q2 rows to the front, :278-279).

    softcap / alibi_slopes: what the flash path does with them (:157-194, :235-275). It runs two attentions
    and merges them by log-sum-exp, which is one softmax over the union of their (capped, biased) scores. The
    window attention biases key k of query i by -slope * (pos_i - k). The second attention stacks ALL query
    rows of the call (every sequence's q1 rows, then the q2 rows) into one sequence of `stack_rows` queries
    against the M meta keys with causal=False, for which flash-attn's ALiBi term is
    -slope * |i + M - stack_rows - j| for stacked query i and meta key j. This function's q1 rows are stacked
    queries stack_row0 .. stack_row0 + Lq - 1 and its q2 rows the last M ones (stack_rows defaults to
    Lq (+ M): this sequence alone)."""
    Lq, Hq, D = q1.shape
    Lk, Hkv, _ = k1.shape
    M = k2.shape[0]
    G = Hq // Hkv
    q_id = Lk - Lq + np.arange(Lq)
    k_id = np.arange(Lk)
    visible = np.ones((Lq, M + Lk), bool)
    win = q_id[:, None] >= k_id[None, :]
    if sliding_window > 0:
        win &= (q_id[:, None] - k_id[None, :]) < sliding_window
    visible[:, M:] = win
    q = q1
    n_stack = stack_rows if stack_rows is not None else Lq + (M if q2 is not None else 0)
    stacked = stack_row0 + np.arange(Lq)                      # place of each row in the second attention's sequence
    window_dist = (q_id[:, None] - k_id[None, :]).astype(np.float64)
    if q2 is not None:
        q = np.concatenate([q1, q2], 0)
        meta_rows = np.concatenate([np.ones((M, M), bool), np.zeros((M, Lk), bool)], 1)
        visible = np.concatenate([visible, meta_rows], 0)
        stacked = np.concatenate([stacked, n_stack - M + np.arange(M)])
        window_dist = np.concatenate([window_dist, np.zeros((M, Lk))], 0)
    meta_dist = np.abs(stacked[:, None] + M - n_stack - np.arange(M)[None, :]).astype(np.float64)
    dist = np.concatenate([meta_dist, window_dist], 1)        # [rows, M + Lk], what a slope multiplies
    k = np.concatenate([k2, k1], 0).astype(np.float64)
    v = np.concatenate([v2, v1], 0).astype(np.float64)
    out = np.zeros((q.shape[0], Hq, D))
    for h in range(Hq):
        bias = None if alibi_slopes is None else -float(alibi_slopes[h]) * dist
        out[:, h] = masked_softmax_attention(q[:, h].astype(np.float64), k[:, h // G], v[:, h // G], ~visible, scale,
                                             softcap=softcap, bias=bias)
    return out
