"""Pins oracle.hf_cache.OracleCache without retyping it: closed forms, an independent
list-of-rows model, and the worked traces of cache.py for BASELINE config 1."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle.hf_cache import OracleCache


def rows(n0, n1, B=1, H=2, D=4):
    """Token rows n0..n1-1; row t of (b, h) is filled with 1000*b + 100*h + t (+0.5 for V)."""
    t = np.arange(n0, n1, dtype=np.float32)[None, None, :, None]
    b = np.arange(B, dtype=np.float32)[:, None, None, None] * 1000
    h = np.arange(H, dtype=np.float32)[None, :, None, None] * 100
    k = np.broadcast_to(b + h + t, (B, H, n1 - n0, D)).copy()
    return k, k + 0.5


def token_ids(x):
    return (x[0, 0, :, 0]).astype(int).tolist()


@pytest.mark.parametrize("prompt,expect_after_prefill,kinds", [
    # the four prompts of config 1 at W=512: what is stored after prefill, and which branch each
    # of the 8 decode steps takes ("cat" grows, "roll" keeps 512 rows)
    (300, list(range(0, 300)), ["cat"] * 8),
    (511, list(range(0, 511)), ["cat"] + ["roll"] * 7),
    (700, list(range(188, 700)), ["roll"] * 8),
    (900, list(range(388, 900)), ["roll"] * 8),
])
def test_config1_traces(prompt, expect_after_prefill, kinds):
    W = 512
    c = OracleCache()
    assert c.get_seq_length(0) == 0
    k, v = rows(0, prompt)
    s = c.update(attn_state=(k, v), layer_idx=0, offset=prompt, cache_kwargs={"window_size": W})
    assert token_ids(s["attn_state"][0]) == expect_after_prefill
    assert c.get_seq_length(0) == prompt
    for t, kind in enumerate(kinds, start=1):
        before = s["attn_state"][0].shape[2]
        k, v = rows(prompt + t - 1, prompt + t)
        s = c.update(attn_state=(k, v), layer_idx=0, offset=1, cache_kwargs={"window_size": W})
        after = s["attn_state"][0].shape[2]
        assert (after == before + 1) if kind == "cat" else (after == before == W)
        n = prompt + t
        assert token_ids(s["attn_state"][0]) == list(range(max(0, n - W), n))  # last min(n, W) rows, in order
        assert np.array_equal(s["attn_state"][1], s["attn_state"][0] + 0.5)
        assert c.get_seq_length(0) == n


class ListModel:
    """Independent model: python lists of token ids, written from the prose description."""

    def __init__(self):
        self.rows = None

    def update(self, new, W):
        if self.rows is None:
            self.rows = list(new[-W:]) if (W is not None and len(new) > W) else list(new)
        elif W is not None and len(self.rows) == W:
            if len(new) > W:
                raise ValueError
            self.rows = self.rows[len(new):] + list(new)
        else:
            self.rows = self.rows + list(new)
        return self.rows


@settings(max_examples=150, deadline=None)
@given(W=st.one_of(st.none(), st.integers(1, 12)), prompt=st.integers(1, 30),
       chunks=st.lists(st.integers(1, 5), min_size=0, max_size=12))
def test_against_list_model(W, prompt, chunks):
    c, m = OracleCache(), ListModel()
    n = 0
    for i, step in enumerate([prompt] + chunks):
        if i > 0 and W is not None and len(m.rows) == W and step > W:
            break  # the reference's slice-assign would raise here; not a case callers produce
        k, v = rows(n, n + step, B=2)
        s = c.update(attn_state=(k, v), layer_idx=0, offset=step, cache_kwargs={"window_size": W})
        exp = m.update(list(range(n, n + step)), W)
        n += step
        assert token_ids(s["attn_state"][0]) == exp
        assert (s["attn_state"][0][1, 1, :, 0] - 1100).astype(int).tolist() == exp
        assert c.get_seq_length(0) == n


def test_overshoot_is_never_trimmed():
    # multi-token append onto a non-full cache overshoots W; the equality test then never fires
    W = 8
    c = OracleCache()
    c.update(attn_state=rows(0, 6), layer_idx=0, offset=6, cache_kwargs={"window_size": W})
    s = c.update(attn_state=rows(6, 10), layer_idx=0, offset=4, cache_kwargs={"window_size": W})
    assert s["attn_state"][0].shape[2] == 10
    s = c.update(attn_state=rows(10, 11), layer_idx=0, offset=1, cache_kwargs={"window_size": W})
    assert token_ids(s["attn_state"][0]) == list(range(11))


def test_counter_only_moves_on_layer0_and_layers_append_in_order():
    c = OracleCache()
    S0 = np.zeros((1, 2, 4, 4), np.float32)
    c.update(recurrent_state=S0, layer_idx=0, offset=5)               # GLA layer 0 bumps the counter
    c.update(attn_state=rows(0, 5), layer_idx=1, offset=5, cache_kwargs={"window_size": 4})
    assert len(c) == 2 and c.get_seq_length(0) == 5 and c.get_seq_length(1) == 5
    assert c.get_seq_length(2) == 0                                   # no entry yet
    S1 = S0 + 1
    st0 = c.update(recurrent_state=S1, layer_idx=0, offset=1)
    assert st0["recurrent_state"] is S1                               # replaced by reference
    c.update(attn_state=rows(5, 6), layer_idx=1, offset=1, cache_kwargs={"window_size": 4})
    assert c.get_seq_length(1) == 6                                   # SWA layer did not add
    assert token_ids(c[1]["attn_state"][0]) == [2, 3, 4, 5]
    with pytest.raises(KeyError):
        c[2]
    conv = (None,)
    assert c.update(conv_state=conv, layer_idx=0, offset=0)["conv_state"] is conv


def test_errors_and_legacy_roundtrip():
    c = OracleCache()
    with pytest.raises(ValueError):
        c.update(attn_state=[rows(0, 1)[0], rows(0, 1)[1]], layer_idx=0, cache_kwargs={})  # list, not tuple
    with pytest.raises(AttributeError):
        OracleCache().update(attn_state=rows(0, 1), layer_idx=0, cache_kwargs=None)          # .get on None
    c = OracleCache()
    c.update(attn_state=rows(0, 3), layer_idx=0, offset=3, cache_kwargs={})
    legacy = c.to_legacy_cache()
    c2 = OracleCache.from_legacy_cache(legacy, seen_tokens=3)
    assert len(c2) == 1 and c2.get_seq_length() == 3 and c2[0] is legacy[0]
    assert c2.get_max_length() is None
    assert [s for s in c2] == list(legacy)
