"""`sliding_window_attention` called the way the reference's two layer files call their cache and
attention, with the function's DEFAULTS (no cache_window_size / window_left overrides):

  flavour="flash"  hf_7B_model/window_attention.py:164-217: cache bounded at W rows
                   (`window_size=W` handed to `Cache.update`), flash window (W, 0): a prompt query
                   sees itself and W keys to its left (W+1 keys), a decode query the W cached rows;
  flavour="sdpa"   hf_7B_model/window_attention_sdpa.py:174-214: no window handed to the cache (it
                   grows without bound), mask of W keys including the query itself.

BASELINE config 1 shapes (28 q / 4 kv heads, D=128, W=512, prompts 300/511/700/900, 8 decode steps),
per sequence and as one left-padded batch, next to OracleCache + the oracle attention of the same
flavour on identical seeded inputs. Cache tensors bit-exact after every step; outputs within 1e-5
(fp32) / 2e-2 (bf16) max-abs."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle.hf_cache import OracleCache

pytestmark = pytest.mark.gpu

HQ, HKV, D, W = 28, 4, 128, 512
PROMPTS = [300, 511, 700, 900]
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def draw(g, B, n, dtype):
    k = torch.randn(B, HKV, n, D, generator=g).to(dtype)
    v = torch.randn(B, HKV, n, D, generator=g).to(dtype)
    q = torch.randn(B, HQ, n, D, generator=g).to(dtype)
    return q, k, v


def oracle_step(flavour, cache, q, k, v, mask):
    """The reference layer's cache + attention slice on numpy (window_attention.py:164-174 /
    window_attention_sdpa.py:174-184, then the flavour's attention)."""
    qn, kn, vn = (t.float().numpy() for t in (q, k, v))
    has = cache.get_seq_length(0) > 0
    kwargs = {"window_size": W} if flavour == "flash" else {}          # sdpa file passes no window_size (:176)
    kc, vc = cache.update(attn_state=(kn.copy(), vn.copy()), layer_idx=0, offset=q.shape[2], cache_kwargs=kwargs)["attn_state"]
    kk, vv = (kc, vc) if has else (kn, vn)
    fn = A.flash_window_attention if flavour == "flash" else A.sdpa_window_attention
    return fn(qn, kk, vv, W, mask)


def product_step(sb, dev, flavour, cache, q, k, v, mask):
    out = sb.sliding_window_attention(q.to(dev), k.to(dev), v.to(dev), W, cache, 0,
                                      attention_mask=None if mask is None else torch.from_numpy(mask).to(dev),
                                      flavour=flavour)
    return out.permute(0, 2, 1, 3).float().cpu().numpy()


def check_cache(prod, orc):
    pk, pv = prod[0]["attn_state"]
    ok, ov = orc[0]["attn_state"]
    assert pk.shape == ok.shape
    assert np.array_equal(pk.float().cpu().numpy(), ok) and np.array_equal(pv.float().cpu().numpy(), ov)
    assert prod.get_seq_length(0) == orc.get_seq_length(0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("flavour", ["flash", "sdpa"])
@pytest.mark.parametrize("prompt", PROMPTS)
def test_default_flavours_per_sequence(sb, dev, prompt, flavour, dtype):
    g = torch.Generator().manual_seed(prompt)
    prod, orc = sb.Cache(), OracleCache()
    q, k, v = draw(g, 1, prompt, dtype)
    ref = oracle_step(flavour, orc, q, k, v, None)
    got = product_step(sb, dev, flavour, prod, q, k, v, None)
    check_cache(prod, orc)
    assert np.abs(got - ref).max() <= TOL[dtype]
    # what the cache holds is the flavour's convention: W rows at most (flash) or everything (sdpa)
    assert prod[0]["attn_state"][0].shape[2] == (min(prompt, W) if flavour == "flash" else prompt)
    for t in range(1, 9):
        q, k, v = draw(g, 1, 1, dtype)
        ref = oracle_step(flavour, orc, q, k, v, None)
        got = product_step(sb, dev, flavour, prod, q, k, v, None)
        check_cache(prod, orc)
        assert prod[0]["attn_state"][0].shape[2] == (min(prompt + t, W) if flavour == "flash" else prompt + t)
        assert np.abs(got - ref).max() <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("flavour", ["flash", "sdpa"])
def test_default_flavours_left_padded_batch(sb, dev, flavour, dtype):
    g = torch.Generator().manual_seed(7)
    L = max(PROMPTS)
    mask = np.zeros((4, L), np.int64)
    for b, n in enumerate(PROMPTS):
        mask[b, L - n:] = 1
    prod, orc = sb.Cache(), OracleCache()
    q, k, v = draw(g, 4, L, dtype)
    ref = oracle_step(flavour, orc, q, k, v, mask)
    got = product_step(sb, dev, flavour, prod, q, k, v, mask)
    check_cache(prod, orc)
    assert np.abs(got - ref).max() <= TOL[dtype]
    for b, n in enumerate(PROMPTS):                       # pad queries: zeros (pad_input / nan_to_num)
        assert (got[b, :, :L - n] == 0).all()
    for t in range(1, 9):
        mask = np.concatenate([mask, np.ones((4, 1), np.int64)], axis=1)
        q, k, v = draw(g, 4, 1, dtype)
        ref = oracle_step(flavour, orc, q, k, v, mask)
        got = product_step(sb, dev, flavour, prod, q, k, v, mask)
        check_cache(prod, orc)
        assert np.abs(got - ref).max() <= TOL[dtype]


def test_the_two_flavours_differ_by_one_key_at_prefill(sb, dev):
    """Guards the convention itself. All scores equal and V zero except at one key j0, so a query's output
    is 1 / (number of visible keys) if it sees j0 and exactly 0 if not: the last prompt query (W keys past
    j0) sees it only under the flash default, the query before it under both, with W+1 and W visible keys."""
    n = W + 40
    j0 = n - 1 - W
    q = torch.zeros(1, HQ, n, D, dtype=torch.bfloat16)
    k = torch.zeros(1, HKV, n, D, dtype=torch.bfloat16)
    v = torch.zeros(1, HKV, n, D, dtype=torch.bfloat16)
    v[:, :, j0] = 1.0
    flash = product_step(sb, dev, "flash", sb.Cache(), q, k, v, None)[0, :, :, 0]
    sdpa = product_step(sb, dev, "sdpa", sb.Cache(), q, k, v, None)[0, :, :, 0]
    assert np.abs(flash[:, n - 1] - 1 / (W + 1)).max() <= 2e-5 and (sdpa[:, n - 1] == 0).all()
    assert np.abs(flash[:, n - 2] - 1 / (W + 1)).max() <= 2e-5 and np.abs(sdpa[:, n - 2] - 1 / W).max() <= 2e-5
    assert (flash[:, n - 1 - W - 1] == 0).all() and (flash[:, :j0] == 0).all()      # causal: queries before j0
