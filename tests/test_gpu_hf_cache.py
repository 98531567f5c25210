"""BASELINE config 1 on the GPU path: drop-in `Cache` + sliding-window attention slice, stepped
next to the oracle (OracleCache + SDPA-style masked softmax) on identical seeded inputs.
B=4, 28 q heads, 4 kv heads, D=128, W=512, fp32, prompts 300/511/700/900, 8 decode steps.
Cache tensors must be bit-exact after every step; attention within 1e-5 max-abs."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle.hf_cache import OracleCache

pytestmark = pytest.mark.gpu

HQ, HKV, D, W = 28, 4, 128, 512
PROMPTS = [300, 511, 700, 900]
ATOL = 1e-5


def draw(g, B, n):
    """K, then V, then Q for n new tokens (the order is part of the fixture definition)."""
    k = torch.randn(B, HKV, n, D, generator=g)
    v = torch.randn(B, HKV, n, D, generator=g)
    q = torch.randn(B, HQ, n, D, generator=g)
    return q, k, v


def oracle_step(cache, q, k, v, layer_idx, mask):
    has = cache.get_seq_length(layer_idx) > 0
    kc, vc = cache.update(attn_state=(k.numpy().copy(), v.numpy().copy()), layer_idx=layer_idx, offset=q.shape[2],
                          cache_kwargs={"window_size": W})["attn_state"]
    kk, vv = (kc, vc) if has else (k.numpy(), v.numpy())
    return A.sdpa_window_attention(q.numpy(), kk, vv, W, mask)       # [B, Hq, Q, D]


def product_step(sb, dev, cache, q, k, v, layer_idx, mask):
    out = sb.sliding_window_attention(q.to(dev), k.to(dev), v.to(dev), W, cache, layer_idx,
                                      attention_mask=None if mask is None else torch.from_numpy(mask).to(dev),
                                      cache_window_size=W, window_left=W - 1)
    return out.permute(0, 2, 1, 3).cpu().numpy()                      # -> [B, Hq, Q, D]


def check_cache(prod, orc, layer_idx):
    pk, pv = prod[layer_idx]["attn_state"]
    ok, ov = orc[layer_idx]["attn_state"]
    assert pk.shape == ok.shape
    assert np.array_equal(pk.cpu().numpy(), ok) and np.array_equal(pv.cpu().numpy(), ov)
    assert prod.get_seq_length(layer_idx) == orc.get_seq_length(layer_idx)


@pytest.mark.parametrize("prompt", PROMPTS)
def test_config1_per_sequence(sb, dev, prompt):
    g = torch.Generator().manual_seed(0)
    prod, orc = sb.Cache(), OracleCache()
    assert prod.get_seq_length(0) == 0
    q, k, v = draw(g, 1, prompt)
    ref = oracle_step(orc, q, k, v, 0, None)
    got = product_step(sb, dev, prod, q, k, v, 0, None)
    check_cache(prod, orc, 0)
    assert np.abs(got - ref).max() <= ATOL
    assert prod[0]["attn_state"][0].shape[2] == min(prompt, W)
    for t in range(1, 9):
        q, k, v = draw(g, 1, 1)
        ref = oracle_step(orc, q, k, v, 0, None)
        got = product_step(sb, dev, prod, q, k, v, 0, None)
        check_cache(prod, orc, 0)
        assert prod.get_seq_length(0) == prompt + t
        assert prod[0]["attn_state"][0].shape[2] == min(prompt + t, W)
        assert np.abs(got - ref).max() <= ATOL


def test_config1_left_padded_batch(sb, dev):
    g = torch.Generator().manual_seed(0)
    L = max(PROMPTS)
    mask = np.zeros((4, L), np.int64)
    for b, n in enumerate(PROMPTS):
        mask[b, L - n:] = 1
    prod, orc = sb.Cache(), OracleCache()
    q, k, v = draw(g, 4, L)
    ref = oracle_step(orc, q, k, v, 0, mask)
    got = product_step(sb, dev, prod, q, k, v, 0, mask)
    check_cache(prod, orc, 0)
    assert np.abs(got - ref).max() <= ATOL
    for b, n in enumerate(PROMPTS):                     # pad queries come out as zeros (nan_to_num)
        assert (got[b, :, :L - n] == 0).all()
    for t in range(1, 9):
        mask = np.concatenate([mask, np.ones((4, 1), np.int64)], axis=1)
        q, k, v = draw(g, 4, 1)
        ref = oracle_step(orc, q, k, v, 0, mask)
        got = product_step(sb, dev, prod, q, k, v, 0, mask)
        check_cache(prod, orc, 0)
        assert np.abs(got - ref).max() <= ATOL


def test_cache_contract_multi_layer_and_quirks(sb, dev):
    """Layer bookkeeping, counter rule, overshoot quirk, unbounded window, compaction over many
    steps and the legacy round trip, each compared with the oracle cache."""
    g = torch.Generator().manual_seed(1)
    prod, orc = sb.Cache(), OracleCache()
    S = torch.zeros(2, HQ, D, D)
    prod.update(recurrent_state=S.to(dev), layer_idx=0, offset=6)
    orc.update(recurrent_state=S.numpy(), layer_idx=0, offset=6)

    def both(n, layer, window, dtype=torch.float32):
        k = torch.randn(2, HKV, n, D, generator=g).to(dtype)
        v = torch.randn(2, HKV, n, D, generator=g).to(dtype)
        prod.update(attn_state=(k.to(dev), v.to(dev)), layer_idx=layer, offset=n, cache_kwargs={"window_size": window})
        orc.update(attn_state=(k.float().numpy(), v.float().numpy()), layer_idx=layer, offset=n, cache_kwargs={"window_size": window})
        pk, pv = prod[layer]["attn_state"]
        ok, ov = orc[layer]["attn_state"]
        assert np.array_equal(pk.float().cpu().numpy(), ok) and np.array_equal(pv.float().cpu().numpy(), ov)

    both(6, 1, 8)            # layer 1: first call
    both(4, 1, 8)            # overshoots the window of 8 -> 10 rows, never trimmed afterwards
    both(1, 1, 8)
    assert prod[1]["attn_state"][0].shape[2] == 11
    both(20, 2, 8)           # layer 2: first call longer than the window -> last 8 rows
    for _ in range(200):     # many rolls: the window walks through the buffer and is compacted
        both(1, 2, 8)
    both(3, 2, 8)            # a 3-token roll
    both(5, 3, None, torch.bfloat16)   # unbounded bf16 layer grows (buffer re-allocation path)
    for _ in range(150):
        both(1, 3, None, torch.bfloat16)
    assert prod.get_seq_length(0) == orc.get_seq_length(0) == 6 and prod.get_seq_length(4) == 0
    assert len(prod) == len(orc) == 4
    with pytest.raises(KeyError):
        prod[4]
    with pytest.raises(ValueError):
        prod.update(attn_state=[S, S], layer_idx=1, cache_kwargs={})
    legacy = prod.to_legacy_cache()
    again = sb.Cache.from_legacy_cache(legacy, seen_tokens=6)
    assert len(again) == 4 and again[2] is legacy[2] and again.get_seq_length(3) == 6 and again.get_max_length() is None
    # a layer adopted from the legacy tuple keeps working (re-homed on its next update)
    k = torch.randn(2, HKV, 1, D, generator=g)
    again.update(attn_state=(k.to(dev), k.to(dev)), layer_idx=2, offset=1, cache_kwargs={"window_size": 8})
    orc.update(attn_state=(k.numpy(), k.numpy()), layer_idx=2, offset=1, cache_kwargs={"window_size": 8})
    assert np.array_equal(again[2]["attn_state"][0].cpu().numpy(), orc[2]["attn_state"][0])
