"""Pins oracle.cpu_path (the torch-CPU restatement bench.py times as `cpu_baseline`) without
retyping it: an independent list-of-rows model of the dense window cache, an explicit
mask-and-softmax loop written from the prose of window_attention_sdpa.py, and the float64
unrolled closed form of the GLA recurrence."""
import math

import numpy as np
import pytest
import torch

from oracle import cpu_path as P


# ---- dense_window_update (hf_7B_model/cache.py:79-89, 94-107) ---------------------------------------
def token_rows(n0, n1, B=2, H=3, D=4):
    """Rows n0..n1-1; K row t of (b, h) holds 1000 b + 100 h + t in every element, V the same + 0.5."""
    t = torch.arange(n0, n1, dtype=torch.float32)[None, None, :, None]
    b = torch.arange(B, dtype=torch.float32)[:, None, None, None] * 1000
    h = torch.arange(H, dtype=torch.float32)[None, :, None, None] * 100
    k = (b + h + t).expand(B, H, n1 - n0, D).contiguous()
    return k, k + 0.5


def ids(x, b=0, h=0):
    return (x[b, h, :, 0] - 1000 * b - 100 * h).round().int().tolist()


class ListModel:
    """Lists of token ids, from the prose: first call keeps the last W; a cache of exactly W rows drops
    its n oldest and takes the n new; any other cache grows."""

    def __init__(self):
        self.rows = None

    def update(self, new, W):
        if self.rows is None:
            self.rows = list(new[-W:]) if (W is not None and len(new) > W) else list(new)
        elif W is not None and len(self.rows) == W:
            self.rows = self.rows[len(new):] + list(new)
        else:
            self.rows = self.rows + list(new)
        return self.rows


@pytest.mark.parametrize("prompt", [300, 511, 700, 900])
def test_dense_window_update_config1_traces(prompt):
    W = 512
    k, v = token_rows(0, prompt)
    ks, vs = P.dense_window_update(None, None, k, v, W)
    m = ListModel()
    assert ids(ks) == m.update(list(range(prompt)), W) == list(range(max(0, prompt - W), prompt))
    for t in range(1, 9):
        k, v = token_rows(prompt + t - 1, prompt + t)
        ks, vs = P.dense_window_update(ks, vs, k, v, W)
        n = prompt + t
        exp = m.update([n - 1], W)
        assert exp == list(range(max(0, n - W), n))        # closed form: the last min(n, W) rows, in order
        for b, h in ((0, 0), (1, 2)):
            assert ids(ks, b, h) == exp
        assert torch.equal(vs, ks + 0.5)                   # V moved exactly as K did


def test_dense_window_update_random_schedules_vs_list_model():
    rng = np.random.default_rng(0)
    for _ in range(200):
        W = None if rng.random() < 0.2 else int(rng.integers(1, 12))
        m, ks, vs, n = ListModel(), None, None, 0
        for i in range(int(rng.integers(1, 12))):
            step = int(rng.integers(1, 30 if i == 0 else 6))
            if i > 0 and W is not None and len(m.rows) == W and step > W:
                break  # the reference's slice-assign would raise: not a case callers produce
            k, v = token_rows(n, n + step)
            ks, vs = P.dense_window_update(ks, vs, k, v, W)
            exp = m.update(list(range(n, n + step)), W)
            n += step
            assert ids(ks) == exp and ids(ks, 1, 1) == exp and torch.equal(vs, ks + 0.5)


def test_dense_window_update_overshoot_is_never_trimmed():
    W = 8
    ks, vs = P.dense_window_update(None, None, *token_rows(0, 6), W)
    ks, vs = P.dense_window_update(ks, vs, *token_rows(6, 10), W)      # 6 != 8: cat -> 10 rows
    assert ks.shape[2] == 10
    ks, vs = P.dense_window_update(ks, vs, *token_rows(10, 11), W)     # 10 != 8: cat again, never evicts
    assert ids(ks) == list(range(11))


# ---- repeat_kv (window_attention_sdpa.py:82-91) -------------------------------------------------------
def test_repeat_kv_is_repeat_interleave_on_the_head_axis():
    x = torch.randn(2, 4, 5, 3, generator=torch.Generator().manual_seed(0))
    assert torch.equal(P.repeat_kv(x, 7), x.repeat_interleave(7, dim=1))
    assert P.repeat_kv(x, 1) is x


# ---- sdpa_window_attention (window_attention_sdpa.py:140-148, 186-214) -------------------------------
def explicit_attention(q, k, v, W, attention_mask):
    """Per (batch, head, query): visible keys by the two rules in words (not after the query, fewer than
    W back, counted from the query's absolute position (K - Q) + i; not a padded key), then a softmax
    written out with math.exp. A query with no visible key gives zeros."""
    B, Hq, Q, D = q.shape
    Hkv, K = k.shape[1], k.shape[2]
    G = Hq // Hkv
    out = np.zeros((B, Hq, Q, D))
    for b in range(B):
        padded = [attention_mask is not None and attention_mask[b, attention_mask.shape[1] - K + j] == 0
                  for j in range(K)]
        for h in range(Hq):
            for i in range(Q):
                pos = (K - Q) + i
                vis = [j for j in range(K) if j <= pos and pos - j < W and not padded[j]]
                if not vis:
                    continue
                s = [float(np.dot(q[b, h, i], k[b, h // G, j])) / math.sqrt(D) for j in vis]
                mx = max(s)
                w = [math.exp(x - mx) for x in s]
                tot = sum(w)
                out[b, h, i] = sum((wj / tot) * v[b, h // G, j] for wj, j in zip(w, vis))
    return out


def test_sdpa_window_attention_vs_explicit_softmax():
    g = torch.Generator().manual_seed(1)
    B, Hq, Hkv, Q, K, D, W = 3, 6, 2, 4, 9, 8, 3
    q = torch.randn(B, Hq, Q, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, Hkv, K, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, Hkv, K, D, generator=g, dtype=torch.float64)
    am = torch.ones(B, K + 3, dtype=torch.int64)
    am[1, :6] = 0          # left padding: the first 3 cached keys of row 1 are pads
    am[2, :10] = 0         # row 2 pads reach into the queries: its first two queries see no key at all
    got = P.sdpa_window_attention(q, k, v, W, am).numpy()
    ref = explicit_attention(q.numpy(), k.numpy(), v.numpy(), W, am.numpy())
    np.testing.assert_allclose(got, ref, rtol=1e-10, atol=1e-12)
    assert (got[2, :, :2] == 0).all() and np.abs(got[2, :, 2:]).min() > 0      # fully masked rows -> exactly 0
    # decode shape (one query at the end), no padding mask, window wider than the cache
    got1 = P.sdpa_window_attention(q[:, :, -1:], k, v, 100, None).numpy()
    ref1 = explicit_attention(q[:, :, -1:].numpy(), k.numpy(), v.numpy(), 100, None)
    np.testing.assert_allclose(got1, ref1, rtol=1e-10, atol=1e-12)


def test_sdpa_window_is_W_keys_including_self():
    # constant scores: the output is the plain mean of the visible V rows, which names them
    B, H, K, D, W = 1, 1, 7, 4, 3
    q = torch.zeros(B, H, 2, D, dtype=torch.float64)
    k = torch.zeros(B, H, K, D, dtype=torch.float64)
    v = torch.arange(K, dtype=torch.float64).view(1, 1, K, 1).expand(B, H, K, D).contiguous()
    out = P.sdpa_window_attention(q, k, v, W)
    # queries sit at absolute positions 5 and 6 and see keys {3,4,5} and {4,5,6}
    np.testing.assert_allclose(out[0, 0, :, 0].numpy(), [4.0, 5.0], rtol=1e-12)


# ---- gla_step (my_fused_recurrent.py:60-80) -----------------------------------------------------------
def test_gla_step_vs_unrolled_closed_form():
    # T steps of gla_step from S_0 against S_T = diag(exp(sum_u g_u)) S_0 + sum_t diag(exp(sum_{u>t} g_u)) k_t^T v_t
    # and o_T = scale * q_T S_T, in float64
    g = torch.Generator().manual_seed(2)
    B, H, T, D = 2, 3, 6, 8
    q, k, v = (torch.randn(B, H, T, D, generator=g) for _ in range(3))
    gate = -torch.rand(B, H, T, D, generator=g) * 0.4
    S0 = torch.randn(B, H, D, D, generator=g) * 0.1
    S = S0.clone()
    for t in range(T):
        o = P.gla_step(q[:, :, t], k[:, :, t], v[:, :, t], gate[:, :, t], S, scale=0.37)
    gd, kd, vd, S0d = gate.double().numpy(), k.double().numpy(), v.double().numpy(), S0.double().numpy()
    for b in range(B):
        for h in range(H):
            ref = np.exp(gd[b, h].sum(0))[:, None] * S0d[b, h]
            for t in range(T):
                ref = ref + np.exp(gd[b, h, t + 1:].sum(0))[:, None] * np.outer(kd[b, h, t], vd[b, h, t])
            np.testing.assert_allclose(S[b, h].numpy(), ref, rtol=2e-5, atol=2e-6)
            np.testing.assert_allclose(o[b, h].numpy(), 0.37 * q[b, h, -1].double().numpy() @ ref, rtol=2e-5, atol=2e-5)


def test_gla_step_special_cases():
    g = torch.Generator().manual_seed(3)
    B, H, D = 2, 2, 8
    q, k, v = (torch.randn(B, H, D, generator=g) for _ in range(3))
    S0 = torch.randn(B, H, D, D, generator=g)
    S = S0.clone()                                        # g = 0: pure accumulation of the outer product
    P.gla_step(q, k, v, torch.zeros(B, H, D), S, scale=1.0)
    torch.testing.assert_close(S, S0 + k[..., :, None] * v[..., None, :])
    gate = -torch.rand(B, H, D, generator=g)
    S = S0.clone()                                        # k = 0: rows (key dims) decay by exp(g)
    P.gla_step(q, torch.zeros_like(k), v, gate, S, scale=1.0)
    torch.testing.assert_close(S, gate.exp()[..., :, None] * S0)
    S = S0.clone()                                        # q = e_3 / scale reads row 3 of the UPDATED state
    e = torch.zeros(B, H, D)
    e[..., 3] = 4.0
    o = P.gla_step(e, k, v, gate, S, scale=0.25)
    torch.testing.assert_close(o, S[..., 3, :])
    S1, S2 = S0.clone(), S0.clone()                       # default scale is D^-0.5
    torch.testing.assert_close(P.gla_step(q, k, v, gate, S1), P.gla_step(q, k, v, gate, S2, scale=D ** -0.5))
    # bf16 inputs are widened before the arithmetic (the state stays fp32)
    S3 = S0.clone()
    P.gla_step(q.bfloat16(), k.bfloat16(), v.bfloat16(), gate, S3)
    S4 = S0.clone()
    P.gla_step(q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float(), gate, S4)
    assert torch.equal(S3, S4)
