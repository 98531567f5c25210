"""Meta-token attention (every query also attends to a few cached rows shared by all sequences):
the log-sum-exp merge op, the log-sum-exp output of the many-query kernel, and the backend's
forward with query2/key2/value2, against the one-softmax oracle statement
(vllm_hymeta/attention/fa_kernel_metatoken.py:372-405). Tolerance: 2e-2 max-abs (bf16)."""
import numpy as np
import pytest
import torch

from oracle import attention as A

pytestmark = pytest.mark.gpu

HQ, HKV, D = 28, 4, 128
TOL = 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_lse_merge_op_vs_oracle(sb, dev, dtype):
    g = torch.Generator().manual_seed(3)
    R, H = 37, 5
    out = torch.randn(R, H, D, generator=g).to(dtype)
    blk = torch.randn(R, H, D, generator=g).to(dtype)
    lse = torch.randn(R, H, generator=g) * 3
    blse = torch.randn(R, H, generator=g) * 3
    lse[2, 1] = float("-inf")           # nothing on the window side: the block side wins
    blse[5, 0] = float("-inf")          # nothing on the block side: unchanged
    lse[7, 3] = blse[7, 3] = float("-inf")
    with np.errstate(invalid="ignore"):     # the -inf rows come out NaN in the plain formula; set below
        ref_o, ref_l = A.lse_merge(out.float().numpy(), lse.numpy().astype(np.float64), blk.float().numpy(),
                                   blse.numpy().astype(np.float64))
    ref_o[2, 1], ref_l[2, 1] = blk[2, 1].float().numpy(), blse[2, 1]
    ref_o[5, 0], ref_l[5, 0] = out[5, 0].float().numpy(), lse[5, 0]
    ref_o[7, 3], ref_l[7, 3] = out[7, 3].float().numpy(), -np.inf
    # strided views: out as a slice of a wider buffer
    wide = torch.zeros(R, H + 2, D, dtype=dtype, device=dev)
    o = wide[:, 1:H + 1]
    o.copy_(out)
    l = lse.clone().to(dev)
    sb.ops.lse_merge(o, l, blk.to(dev), blse.to(dev))
    tol = {torch.bfloat16: 2e-2, torch.float16: 4e-3, torch.float32: 1e-5}[dtype]
    assert np.abs(o.float().cpu().numpy() - ref_o).max() <= tol
    got_l = l.cpu().numpy()
    finite = np.isfinite(ref_l)
    assert np.abs(got_l[finite] - ref_l[finite]).max() <= 1e-5
    assert np.isneginf(got_l[~finite]).all()
    assert (wide[:, 0] == 0).all() and (wide[:, H + 1] == 0).all()


def test_prefill_kernel_lse_vs_oracle(sb, dev):
    g = torch.Generator().manual_seed(4)
    qlens, klens, wl = [70, 5, 130], [70, 40, 200], 47
    Tq, Tk = sum(qlens), sum(klens)
    q = torch.randn(Tq, HQ, D, generator=g).bfloat16()
    k = torch.randn(Tk, HKV, D, generator=g).bfloat16()
    v = torch.randn(Tk, HKV, D, generator=g).bfloat16()
    cu_k = np.concatenate([[0], np.cumsum(klens)])
    out, lse = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=qlens, seq_lens_k=klens,
                                            kv_start=torch.tensor(cu_k[:-1], dtype=torch.int64, device=dev),
                                            window_left=wl, return_lse=True)
    lse = lse.cpu().numpy()
    qf, kf = q.float().numpy().astype(np.float64), k.float().numpy().astype(np.float64)
    scale = D ** -0.5
    t = 0
    for s, (nq, nk) in enumerate(zip(qlens, klens)):
        for j in range(nq):
            pos = nk - nq + j
            ks = slice(cu_k[s] + max(0, pos - wl), cu_k[s] + pos + 1)
            for h in (0, 9, 27):
                sc = kf[ks, h // 7] @ qf[t + j, h] * scale
                ref = np.log(np.exp(sc - sc.max()).sum()) + sc.max()
                assert abs(lse[t + j, h] - ref) <= 2e-3, (s, j, h)
        t += nq


def expected_with_meta(q, hist_k, hist_v, k2, v2, wl, q2=None):
    """q [n, Hq, D] = the last n tokens of a sequence whose keys so far are hist_k/hist_v."""
    return A.metatoken_attention(q, q2, hist_k, k2, hist_v, v2, D ** -0.5, wl + 1)


@pytest.mark.parametrize("M", [128, 32])
def test_backend_forward_with_meta_tokens(sb, dev, M):
    """Prompt step with query2 (meta outputs first), chunked second prompt + decodes, then decode
    steps, all with key2/value2; cache contents are those of the plain path."""
    bs, wl, nb = 16, 40, 64
    g = torch.Generator().manual_seed(M)
    runner = sb.runner.SwaCacheRunner(1, nb, bs, wl, HKV, D, torch.bfloat16, dev, max_seqs=3, max_chunk_tokens=128)
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, wl + 1, "auto", num_meta_tokens=M)
    k2 = torch.randn(M, HKV, D, generator=g).bfloat16()
    v2 = torch.randn(M, HKV, D, generator=g).bfloat16()
    q2 = torch.randn(M, HQ, D, generator=g).bfloat16()
    k2n, v2n, q2n = (x.float().numpy() for x in (k2, v2, q2))
    hist = {}

    def step(prompts, decodes, chunked=False, with_q2=False):
        T = sum(n for _, n in prompts) + len(decodes)
        q = torch.randn(T, HQ, D, generator=g).bfloat16()
        k = torch.randn(T, HKV, D, generator=g).bfloat16()
        v = torch.randn(T, HKV, D, generator=g).bfloat16()
        meta = runner.build_step(prompts, decodes, chunked_prefill=chunked)
        extra = M if with_q2 else 0
        out = torch.full((T + extra, HQ, D), float("nan"), dtype=torch.bfloat16, device=dev)
        impl.forward(None, q.to(dev), k.to(dev), v.to(dev), q2.to(dev) if with_q2 else None, k2.to(dev), v2.to(dev),
                     runner.kv_caches[0], meta, output=out)
        got = out.float().cpu().numpy()
        assert not np.isnan(got).any()
        t = 0
        for sid, n in list(prompts) + [(s, 1) for s in decodes]:
            hk, hv = hist.get(sid, (np.zeros((0, HKV, D), np.float32), np.zeros((0, HKV, D), np.float32)))
            hk = np.concatenate([hk, k[t:t + n].float().numpy()]); hv = np.concatenate([hv, v[t:t + n].float().numpy()])
            hist[sid] = (hk, hv)
            ref = expected_with_meta(q[t:t + n].float().numpy(), hk, hv, k2n, v2n, wl)
            assert np.abs(got[extra + t:extra + t + n] - ref).max() <= TOL, (sid, n)
            t += n
        if with_q2:
            ref2 = A.metatoken_attention(q2n[:0], q2n, np.zeros((0, HKV, D)), k2n, np.zeros((0, HKV, D)), v2n, D ** -0.5, 0)
            assert np.abs(got[:M] - ref2).max() <= TOL

    for sid in (0, 1, 2):
        runner.add_seq(sid)
    step([(0, 30), (1, 100)], [], with_q2=True)             # plain prompts, in-flight keys
    step([(2, 50)], [0, 1], chunked=True)                   # chunked prompt from the paged cache + decodes
    for _ in range(bs + 2):
        step([], [0, 1, 2])                                 # pure decode steps (fused append)


def test_meta_token_argument_errors(sb, dev):
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, 41, "auto", num_meta_tokens=32)
    runner = sb.runner.SwaCacheRunner(1, 16, 16, 40, HKV, D, torch.bfloat16, dev, max_seqs=1, max_chunk_tokens=64)
    runner.add_seq(0)
    meta = runner.build_step([(0, 8)], [])
    q = torch.zeros(8, HQ, D, dtype=torch.bfloat16, device=dev)
    kv = torch.zeros(8, HKV, D, dtype=torch.bfloat16, device=dev)
    k2 = torch.zeros(32, HKV, D, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(8, HQ, D, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        impl.forward(None, q, kv, kv, None, k2, None, runner.kv_caches[0], meta, output=out)
    with pytest.raises(AssertionError):
        impl.forward(None, q, kv, kv, None, k2[:16], k2[:16], runner.kv_caches[0], meta, output=out)
    with pytest.raises(ValueError):
        sb.ops.lse_merge(out, torch.zeros(8, HQ, device=dev), out[:4], torch.zeros(8, HQ, device=dev))
