"""Committed golden vectors (tests/golden/cache_path_v1.npz, written by tests/golden/make_fixtures.py):
the oracle must still reproduce them (CPU), and the HIP path must match them through the C ABI (GPU).
Integer / byte results bit-exact; attention within 2e-2 (bf16 kernels) of the stored fp64-computed values."""
import os

import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle import gla as G
from oracle import paged as P
from oracle.hf_cache import OracleCache

F = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cache_path_v1.npz"))


def f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def bf16_tensor(bits, dev):
    return torch.from_numpy(bits.astype(np.int16)).view(torch.bfloat16).to(dev)


def run_script(model_add, model_free, model_append):
    slots = []
    for op, s, n, chunked in F["pg_script"].tolist():
        if op == 0:
            model_add(s)
        elif op == 3:
            model_free(s)
        else:
            slots += list(model_append(s, n, op == 1, bool(chunked)))
    return slots


# ---------------------------------------------------------------- oracle vs fixtures (CPU)
def test_oracle_hf_cache_reproduces_fixture():
    cache, t = OracleCache(), 0
    W = int(F["hf_window"])
    for i, n in enumerate(F["hf_steps"].tolist()):
        k, v = F["hf_stream_k"][:, :, t:t + n].copy(), F["hf_stream_v"][:, :, t:t + n].copy()
        st = cache.update(attn_state=(k, v), layer_idx=0, offset=n, cache_kwargs={"window_size": W})["attn_state"]
        assert np.array_equal(st[0], F[f"hf_k_after_{i}"]) and np.array_equal(st[1], F[f"hf_v_after_{i}"])
        t += n
    assert cache.get_seq_length(0) == int(F["hf_seen_tokens"])


def test_oracle_block_model_reproduces_fixture():
    nb, bs, wl = F["pg_params"].tolist()
    m = P.WindowCacheModel(nb, bs, wl)
    slots = run_script(m.add_seq, m.free_seq, lambda s, n, p, c: m.append_tokens(s, n, p, store_all=c))
    assert slots == F["pg_slots"].tolist()
    assert m.free == F["pg_free"].tolist()
    for s in (1, 2):
        table, n, first = m.view(s)
        assert table + [n, first] == F[f"pg_view_{s}"].tolist()


def test_oracle_attention_and_gla_reproduce_fixture():
    D = 128
    o, lse = A.paged_decode_attention(f32(F["dec_q"]), f32(F["dec_k_cache"]), f32(F["dec_v_cache"]), F["dec_tables"],
                                      F["dec_lens"].tolist(), D ** -0.5, int(F["dec_window_left"]), return_lse=True)
    assert np.abs(o - F["dec_out"]).max() <= 1e-6 and np.abs(lse - F["dec_lse"]).max() <= 1e-5
    cu = np.concatenate([[0], np.cumsum(F["pre_query_lens"])])
    po = A.varlen_window_attention(f32(F["pre_q"]), f32(F["pre_k"]), f32(F["pre_v"]), cu, cu, D ** -0.5,
                                   int(F["pre_window_left"]))
    assert np.abs(po - F["pre_out"]).max() <= 1e-6
    st = F["gla_state"].astype(np.float64).copy()
    go = G.gla_step(f32(F["gla_q"]), f32(F["gla_k"]), f32(F["gla_v"]), F["gla_g"], st)
    assert np.abs(go - F["gla_out"]).max() <= 1e-6
    assert np.abs(st[0, 0].sum(1) - F["gla_state_rowsum"]).max() <= 1e-5
    assert np.abs(st[0, 0].sum(0) - F["gla_state_colsum"]).max() <= 1e-5


def test_host_block_manager_reproduces_fixture(sb):
    nb, bs, wl = F["pg_params"].tolist()
    m = sb.WindowBlockManager(nb, bs, wl, max_seqs=4, max_chunk_tokens=80)
    slots = run_script(m.add_seq, m.free_seq, lambda s, n, p, c: m.append_tokens(s, n, p, store_all=c))
    assert slots == F["pg_slots"].tolist()
    assert m.free_stack() == F["pg_free"].tolist()


# ---------------------------------------------------------------- HIP path vs fixtures (GPU)
@pytest.mark.gpu
def test_gpu_hf_cache_matches_fixture(sb, dev):
    cache, t = sb.Cache(), 0
    W = int(F["hf_window"])
    for i, n in enumerate(F["hf_steps"].tolist()):
        k = torch.from_numpy(F["hf_stream_k"][:, :, t:t + n].copy()).to(dev)
        v = torch.from_numpy(F["hf_stream_v"][:, :, t:t + n].copy()).to(dev)
        st = cache.update(attn_state=(k, v), layer_idx=0, offset=n, cache_kwargs={"window_size": W})["attn_state"]
        assert np.array_equal(st[0].cpu().numpy(), F[f"hf_k_after_{i}"])
        assert np.array_equal(st[1].cpu().numpy(), F[f"hf_v_after_{i}"])
        t += n
    assert cache.get_seq_length(0) == int(F["hf_seen_tokens"])


@pytest.mark.gpu
def test_gpu_attention_matches_fixture(sb, dev):
    out, lse = sb.ops.swa_decode_attention(
        bf16_tensor(F["dec_q"], dev), bf16_tensor(F["dec_k_cache"], dev), bf16_tensor(F["dec_v_cache"], dev),
        torch.from_numpy(F["dec_lens"]).to(dev), block_table=torch.from_numpy(F["dec_tables"]).to(dev),
        window_left=int(F["dec_window_left"]), return_lse=True)
    assert np.abs(out.float().cpu().numpy() - F["dec_out"]).max() <= 2e-2
    assert np.abs(lse.cpu().numpy() - F["dec_lse"]).max() <= 1e-3
    pre = sb.ops.swa_prefill_attention(bf16_tensor(F["pre_q"], dev), bf16_tensor(F["pre_k"], dev),
                                       bf16_tensor(F["pre_v"], dev), query_lens=F["pre_query_lens"].tolist(),
                                       window_left=int(F["pre_window_left"]))
    assert np.abs(pre.float().cpu().numpy() - F["pre_out"]).max() <= 2e-2


@pytest.mark.gpu
def test_gpu_gla_matches_fixture(sb, dev):
    state = torch.from_numpy(F["gla_state"].copy()).to(dev)
    q, k, v = (bf16_tensor(F[n], dev).view(1, 1, 1, 128) for n in ("gla_q", "gla_k", "gla_v"))
    g = torch.from_numpy(F["gla_g"]).to(dev).view(1, 1, 1, 128)
    o = sb.ops.gla_recurrent(q, k, v, g, state).float().cpu().numpy().reshape(128)
    ref = F["gla_out"].reshape(128)
    assert (np.abs(o - ref) <= 2e-2 + np.abs(ref) * 2.0 ** -8).all()
    s = state.cpu().numpy()[0, 0].astype(np.float64)
    scale = max(1.0, np.abs(s).max())
    assert np.abs(s.sum(1) - F["gla_state_rowsum"]).max() <= 1e-4 * scale * 128
    assert np.abs(np.diag(s) - F["gla_state_diag"]).max() <= 1e-4 * scale
