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


# ---------------------------------------------------------------- later paths (cache_path_v2_ext.npz)
X = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cache_path_v2_ext.npz"))


def test_oracle_reproduces_extension_fixture():
    from oracle import quant as Q
    codes, scale = Q.quantize_rows(f32(X["i8_rows"]))
    assert np.array_equal(codes, X["i8_codes"]) and np.array_equal(scale, X["i8_scales"])
    assert np.array_equal(Q.dequantize_rows(codes, scale, "bf16"), X["i8_dequant_bf16"])
    mo = A.metatoken_attention(*(f32(X[n]) for n in ("mt_q1", "mt_q2", "mt_k1", "mt_k2", "mt_v1", "mt_v2")),
                               128 ** -0.5, int(X["mt_sliding_window"]))
    np.testing.assert_allclose(mo, X["mt_out"], rtol=1e-6, atol=1e-6)
    go, gs = G.gla_recurrent(f32(X["glp_q"]), f32(X["glp_k"]), f32(X["glp_v"]), X["glp_g"], X["glp_state0"].astype(np.float64))
    np.testing.assert_allclose(go, X["glp_out"], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(gs[0, 0].sum(1), X["glp_state_rowsum"], rtol=1e-5, atol=1e-5)
    o, lse = A.paged_decode_attention(f32(X["rag_q"]), f32(X["rag_k_cache"]), f32(X["rag_v_cache"]), X["rag_tables"],
                                      X["rag_lens"].tolist(), 128 ** -0.5, -1, return_lse=True)
    np.testing.assert_allclose(o, X["rag_out"], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(lse, X["rag_lse"], rtol=1e-6, atol=1e-6)


@pytest.mark.gpu
def test_gpu_int8_and_metatoken_match_extension_fixture(sb, dev):
    rows = bf16_tensor(X["i8_rows"], dev)
    T, H, D = rows.shape
    kv, sc = sb.ops.alloc_int8_kv_cache(1, 16, H, D, dev)
    slots = torch.arange(T, dtype=torch.int64, device=dev)
    sb.ops.kv_append_int8(rows, rows, kv[0], kv[1], sc[0], sc[1], slots)
    assert np.array_equal(kv[0, 0, :T].cpu().numpy(), X["i8_codes"])                       # bit-exact codes
    assert np.array_equal(sc[0, 0, :, :T].cpu().numpy().T, X["i8_scales"])                 # and scales
    assert np.array_equal(sb.ops.quantize_sym(rows).float().cpu().numpy(), X["i8_dequant_bf16"])
    # meta tokens: window attention of the 5 queries (as rows of the single-query kernel over the dense keys),
    # merged with their attention over the meta tokens; the meta tokens' own queries see meta tokens only
    q1, q2, k1, v1, k2, v2 = (bf16_tensor(X[n], dev) for n in ("mt_q1", "mt_q2", "mt_k1", "mt_v1", "mt_k2", "mt_v2"))
    Lq, Lk, W = q1.shape[0], k1.shape[0], int(X["mt_sliding_window"])
    seq_lens = torch.arange(Lk - Lq + 1, Lk + 1, dtype=torch.int32, device=dev)
    out, lse = sb.ops.swa_decode_attention(
        q1, k1, v1, seq_lens, kv_start=torch.zeros(1, dtype=torch.int64, device=dev),
        row_seq=torch.zeros(Lq, dtype=torch.int32, device=dev), kv_strides=(0, k1.stride(0), k1.stride(1)),
        num_kv_heads=k1.shape[1], window_left=W - 1, return_lse=True, max_seq_len=Lk)
    mo, ml = sb.ops.meta_token_attention(q1, k2, v2)
    sb.ops.lse_merge(out, lse, mo, ml)
    own = sb.ops.meta_token_attention(q2, k2, v2)[0]
    got = torch.cat([out, own]).float().cpu().numpy()
    assert np.abs(got - X["mt_out"]).max() <= 2e-2


@pytest.mark.gpu
def test_gpu_gla_prompt_and_ragged_decode_match_extension_fixture(sb, dev):
    q, k, v = (bf16_tensor(X[n], dev) for n in ("glp_q", "glp_k", "glp_v"))
    g = torch.from_numpy(X["glp_g"]).to(dev)
    for vector_only in (False, True):                        # matrix-core block form and step-by-step kernel
        state = torch.from_numpy(X["glp_state0"].copy()).to(dev)
        o = sb.ops.gla_recurrent(q, k, v, g, state, vector_only=vector_only).float().cpu().numpy()
        assert (np.abs(o - X["glp_out"]) <= 2e-2 + np.abs(X["glp_out"]) * 2.0 ** -8).all(), vector_only
        s = state.cpu().numpy()[0, 0].astype(np.float64)
        top = float(X["glp_state_absmax"])
        assert np.abs(np.diag(s) - X["glp_state_diag"]).max() <= 1e-4 * top
        assert np.abs(s.sum(1) - X["glp_state_rowsum"]).max() <= 1e-4 * top * 128
    lens = torch.from_numpy(X["rag_lens"]).to(dev)
    for balanced in (False, True):
        out, lse = sb.ops.swa_decode_attention(
            bf16_tensor(X["rag_q"], dev), bf16_tensor(X["rag_k_cache"], dev), bf16_tensor(X["rag_v_cache"], dev), lens,
            block_table=torch.from_numpy(X["rag_tables"]).to(dev), window_left=-1, return_lse=True, n_split=3,
            balanced=balanced)
        assert np.abs(out.float().cpu().numpy() - X["rag_out"]).max() <= 2e-2, balanced
        assert np.abs(lse.cpu().numpy() - X["rag_lse"]).max() <= 1e-3, balanced
