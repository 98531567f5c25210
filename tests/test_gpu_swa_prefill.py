"""Many-query causal sliding-window attention (prefill kernel) vs the float64 oracle.
Tolerance (BASELINE): max-abs 2e-2 for bf16 (5e-3 for fp16) against fp64 mathematics on the same
bf16/fp16 inputs."""
import numpy as np
import pytest
import torch

from oracle import attention as A

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}


def dense_problem(query_lens, ctx_lens, Hq, Hkv, D, dtype, seed, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    Tq = sum(query_lens)
    lens_k = [a + b for a, b in zip(query_lens, ctx_lens)]
    Tk = sum(lens_k)
    q = (torch.randn(Tq, Hq, D, generator=g) * spread).to(dtype)
    k = (torch.randn(Tk, Hkv, D, generator=g) * spread).to(dtype)
    v = torch.randn(Tk, Hkv, D, generator=g).to(dtype)
    cu_q = np.concatenate([[0], np.cumsum(query_lens)])
    cu_k = np.concatenate([[0], np.cumsum(lens_k)])
    return q, k, v, lens_k, cu_q, cu_k


def check(out, q, k, v, cu_q, cu_k, scale, wl, tol):
    ref = A.varlen_window_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), cu_q, cu_k, scale, wl)
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    err = np.abs(got - ref).max()
    assert err <= tol, f"max abs err {err}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hq,Hkv", [(28, 4), (8, 8), (8, 2), (6, 2), (5, 1)])
@pytest.mark.parametrize("wl", [-1, 0, 1, 31, 64, 100])
def test_prompt_prefill_vs_oracle(sb, dev, dtype, Hq, Hkv, wl):
    """Plain prompts (keys = the step's own tokens): ragged lengths around the 16/32/64 boundaries."""
    D = 128
    query_lens = [1, 15, 16, 17, 33, 64, 65, 127, 130]
    q, k, v, lens_k, cu_q, cu_k = dense_problem(query_lens, [0] * len(query_lens), Hq, Hkv, D, dtype, seed=Hq + wl)
    scale = D ** -0.5
    out = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=query_lens, window_left=wl,
                                       scale=scale)
    check(out, q, k, v, cu_q, cu_k, scale, wl, TOL[dtype])


@pytest.mark.parametrize("wl", [-1, 50, 256])
def test_dense_context_offsets(sb, dev, wl):
    """Queries at the end of longer key sequences (multi-token decode over a dense cache)."""
    D, Hq, Hkv = 128, 28, 4
    query_lens = [3, 64, 20, 1, 70]
    ctx = [200, 5, 0, 77, 300]
    q, k, v, lens_k, cu_q, cu_k = dense_problem(query_lens, ctx, Hq, Hkv, D, torch.bfloat16, seed=wl + 3)
    out = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=query_lens, seq_lens_k=lens_k,
                                       kv_start=torch.tensor(cu_k[:-1], dtype=torch.int64, device=dev),
                                       window_left=wl, scale=D ** -0.5)
    check(out, q, k, v, cu_q, cu_k, D ** -0.5, wl, 2e-2)


@pytest.mark.parametrize("bs", [16, 32, 48, 256])
@pytest.mark.parametrize("wl", [-1, 40, 300])
def test_paged_chunked_prefill_vs_oracle(sb, dev, bs, wl):
    """Chunked prefill: keys (context + the chunk) live in the paged cache in a shuffled block order."""
    D, Hq, Hkv = 128, 28, 4
    query_lens = [64, 10, 130, 1]
    ctx = [100, 0, 515, 33]
    dtype = torch.bfloat16
    q, k, v, lens_k, cu_q, cu_k = dense_problem(query_lens, ctx, Hq, Hkv, D, dtype, seed=bs + wl)
    g = torch.Generator().manual_seed(9)
    need = [(n + bs - 1) // bs for n in lens_k]
    nb = sum(need) + 3
    perm = torch.randperm(nb, generator=g)
    kc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype)   # stale rows hold finite garbage
    vc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype)
    tables = torch.zeros(len(lens_k), max(need), dtype=torch.int32)
    p = 0
    for s, n in enumerate(need):
        tables[s, :n] = perm[p:p + n]; p += n
        for i in range(lens_k[s]):
            blk = int(tables[s, i // bs])
            kc[blk, i % bs] = k[cu_k[s] + i]
            vc[blk, i % bs] = v[cu_k[s] + i]
    out = sb.ops.swa_prefill_attention(q.to(dev), kc.to(dev), vc.to(dev), query_lens=query_lens, seq_lens_k=lens_k,
                                       block_table=tables.to(dev), window_left=wl, scale=D ** -0.5)
    check(out, q, k, v, cu_q, cu_k, D ** -0.5, wl, 2e-2)


def test_growing_scores_raise_the_reference(sb, dev):
    """Keys whose scores keep growing along the sequence force the softmax reference point up many
    times (the rescale path outside the chunk loop), including jumps far above the raise threshold."""
    D, Hq, Hkv = 128, 8, 2
    L = 300
    g = torch.Generator().manual_seed(5)
    q = torch.randn(L, Hq, D, generator=g).abs()
    k = torch.randn(L, Hkv, D, generator=g).abs() * torch.linspace(0.05, 3.0, L)[:, None, None]
    k[150:] *= 2.0
    v = torch.randn(L, Hkv, D, generator=g)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    cu = np.array([0, L])
    for wl in (-1, 100):
        out = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=[L], window_left=wl,
                                           scale=D ** -0.5)
        check(out, q, k, v, cu, cu, D ** -0.5, wl, 2e-2)


def test_matches_decode_kernel_row_by_row(sb, dev):
    """The many-query kernel and the single-query kernel agree on the same paged cache."""
    D, Hq, Hkv, bs, wl = 128, 28, 4, 16, 90
    L = 200
    g = torch.Generator().manual_seed(11)
    nb = (L + bs - 1) // bs
    kc = torch.randn(nb, bs, Hkv, D, generator=g).bfloat16().to(dev)
    vc = torch.randn(nb, bs, Hkv, D, generator=g).bfloat16().to(dev)
    q = torch.randn(L, Hq, D, generator=g).bfloat16().to(dev)
    table = torch.arange(nb, dtype=torch.int32, device=dev)[None]
    pre = sb.ops.swa_prefill_attention(q, kc, vc, query_lens=[L], block_table=table, window_left=wl)
    dec = sb.ops.swa_decode_attention(q, kc, vc, torch.arange(1, L + 1, dtype=torch.int32, device=dev),
                                      block_table=table, row_seq=torch.zeros(L, dtype=torch.int32, device=dev),
                                      window_left=wl)
    assert (pre.float() - dec.float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("wl", [-1, 70])
def test_key_lo_hides_left_padding(sb, dev, wl):
    """Keys below key_lo are invisible; queries inside the padding get zeros."""
    D, Hq, Hkv = 128, 8, 2
    lens = [100, 64, 130]
    pads = [0, 63, 77]
    g = torch.Generator().manual_seed(21)
    T = sum(lens)
    q = torch.randn(T, Hq, D, generator=g).bfloat16()
    k = torch.randn(T, Hkv, D, generator=g).bfloat16()
    v = torch.randn(T, Hkv, D, generator=g).bfloat16()
    out = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=lens, window_left=wl,
                                       key_lo=torch.tensor(pads, dtype=torch.int32, device=dev)).float().cpu().numpy()
    start = 0
    for n, pad in zip(lens, pads):
        sl = slice(start + pad, start + n)                      # the real tokens form their own sequence
        ref = A.varlen_window_attention(q[sl].float().numpy(), k[sl].float().numpy(), v[sl].float().numpy(),
                                        [0, n - pad], [0, n - pad], D ** -0.5, wl)
        assert np.abs(out[sl] - ref).max() <= 2e-2
        assert (out[start:start + pad] == 0).all()
        start += n


def test_hf_layer_prompt_bf16_left_padded(sb, dev):
    """The HuggingFace-side layer slice routes bf16 prompts through the many-query kernel:
    left-padded batch, window 512, then cached decode steps (single-query kernel)."""
    from oracle.hf_cache import OracleCache
    HQ, HKV, D, W = 28, 4, 128, 512
    prompts = [300, 511, 700, 900]
    L = max(prompts)
    g = torch.Generator().manual_seed(0)
    mask = np.zeros((4, L), np.int64)
    for b, n in enumerate(prompts):
        mask[b, L - n:] = 1
    prod, orc = sb.Cache(), OracleCache()
    for step in range(3):
        n = L if step == 0 else 1
        k = torch.randn(4, HKV, n, D, generator=g).bfloat16()
        v = torch.randn(4, HKV, n, D, generator=g).bfloat16()
        q = torch.randn(4, HQ, n, D, generator=g).bfloat16()
        if step:
            mask = np.concatenate([mask, np.ones((4, 1), np.int64)], axis=1)
        has = orc.get_seq_length(0) > 0
        kc, vc = orc.update(attn_state=(k.float().numpy(), v.float().numpy()), layer_idx=0, offset=n,
                            cache_kwargs={"window_size": W})["attn_state"]
        kk, vv = (kc, vc) if has else (k.float().numpy(), v.float().numpy())
        ref = A.sdpa_window_attention(q.float().numpy(), kk, vv, W, mask)
        got = sb.sliding_window_attention(q.to(dev), k.to(dev), v.to(dev), W, prod, 0,
                                          attention_mask=torch.from_numpy(mask).to(dev), cache_window_size=W,
                                          window_left=W - 1).permute(0, 2, 1, 3).float().cpu().numpy()
        assert np.abs(got - ref).max() <= 2e-2
        if step == 0:
            for b, n_real in enumerate(prompts):
                assert (got[b, :, :L - n_real] == 0).all()


def test_prefill_argument_errors(sb, dev):
    q = torch.zeros(4, 8, 128, dtype=torch.bfloat16, device=dev)
    kv = torch.zeros(4, 2, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        sb.ops.swa_prefill_attention(q, kv, kv, query_lens=[3])            # lengths do not cover q
    with pytest.raises(ValueError):
        sb.ops.swa_prefill_attention(q, kv, kv, query_lens=[4], seq_lens_k=[2])   # fewer keys than queries
    with pytest.raises(NotImplementedError):
        sb.ops.swa_prefill_attention(q.float(), kv.float(), kv.float(), query_lens=[4])
    q64 = torch.zeros(4, 8, 64, dtype=torch.bfloat16, device=dev)
    kv64 = torch.zeros(4, 2, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(NotImplementedError):
        sb.ops.swa_prefill_attention(q64, kv64, kv64, query_lens=[4])
    out = sb.ops.swa_prefill_attention(q[:0], kv, kv, query_lens=[])       # empty step
    assert out.shape == (0, 8, 128)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_vs_oracle(sb, dev, seed):
    """Seeded random cases across what the kernel specialises on: GQA group (1..9: launches of 4, 3, 2 and 1 heads,
    double- and single-block wavefronts), dtype, paged (block sizes 16/32/48/64/128, shuffled tables, garbage in
    stale rows) or in-flight keys, window, ragged query and context lengths around the 16/32/64 boundaries,
    optional meta rows, optional soft cap / ALiBi."""
    r = np.random.default_rng(1000 + seed)
    D = 128
    Hkv = int(r.choice([1, 2, 4]))
    G = int(r.integers(1, 10))
    Hq = Hkv * G
    dtype = torch.bfloat16 if r.random() < 0.7 else torch.float16
    S = int(r.integers(1, 6))
    query_lens = [int(r.choice([1, 2, 15, 16, 17, 31, 33, 63, 64, 65, 100, 129, 200])) for _ in range(S)]
    paged = r.random() < 0.6
    ctx = [int(r.choice([0, 1, 31, 32, 77, 300])) if paged else 0 for _ in range(S)]
    wl = int(r.choice([-1, 0, 5, 31, 32, 63, 64, 100, 257]))
    use_meta = r.random() < 0.25
    use_opts = (not use_meta) and r.random() < 0.3
    q, k, v, lens_k, cu_q, cu_k = dense_problem(query_lens, ctx, Hq, Hkv, D, dtype, seed=seed, spread=1.5 if use_opts else 1.0)
    g = torch.Generator().manual_seed(seed)
    kw = {}
    slopes = None
    softcap = 0.0
    if use_opts:
        slopes = [float(2.0 ** (-8.0 * (h + 1) / Hq)) for h in range(Hq)]
        softcap = 2.0
        kw.update(softcap=softcap, alibi_slopes=torch.tensor(slopes, device=dev))
    M = 0
    if use_meta:
        M = int(r.choice([1, 31, 32, 100]))
        mk = torch.randn(M, Hkv, D, generator=g).to(dtype); mv = torch.randn(M, Hkv, D, generator=g).to(dtype)
        kw.update(meta_k=mk.to(dev), meta_v=mv.to(dev))
    scale = D ** -0.5
    if paged:
        bs = int(r.choice([16, 32, 48, 64, 128]))
        need = [(n + bs - 1) // bs for n in lens_k]
        nb = sum(need) + 2
        perm = torch.randperm(nb, generator=g)
        kc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype); vc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype)
        tables = torch.zeros(S, max(need), dtype=torch.int32)
        p = 0
        for s, n in enumerate(need):
            tables[s, :n] = perm[p:p + n]; p += n
            for i in range(lens_k[s]):
                kc[int(tables[s, i // bs]), i % bs] = k[cu_k[s] + i]
                vc[int(tables[s, i // bs]), i % bs] = v[cu_k[s] + i]
        out = sb.ops.swa_prefill_attention(q.to(dev), kc.to(dev), vc.to(dev), query_lens=query_lens, seq_lens_k=lens_k,
                                           block_table=tables.to(dev), window_left=wl, scale=scale, **kw)
    else:
        out = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=query_lens, window_left=wl,
                                           scale=scale, **kw)
    qn, kn, vn = q.float().numpy(), k.float().numpy(), v.float().numpy()
    if use_meta:   # one softmax over [meta rows | window]: the oracle's merged form, query by query
        ref = np.zeros((qn.shape[0], Hq, D))
        for s in range(S):
            Lq, Lk = query_lens[s], lens_k[s]
            for j in range(Lq):
                pos = Lk - Lq + j
                lo = 0 if wl < 0 else max(0, pos - wl)
                for h in range(Hq):
                    kk = np.concatenate([mk.float().numpy()[:, h // G], kn[cu_k[s] + lo:cu_k[s] + pos + 1, h // G]])
                    vv = np.concatenate([mv.float().numpy()[:, h // G], vn[cu_k[s] + lo:cu_k[s] + pos + 1, h // G]])
                    ref[cu_q[s] + j, h] = A.masked_softmax_attention(qn[cu_q[s] + j, h][None], kk, vv,
                                                                     np.zeros((1, len(kk)), bool), scale)[0]
    else:
        ref = A.varlen_window_attention(qn, kn, vn, cu_q, cu_k, scale, wl, softcap=softcap, alibi_slopes=slopes)
    err = np.abs(out.float().cpu().numpy() - ref).max()
    assert err <= TOL[dtype], (err, dict(Hq=Hq, Hkv=Hkv, dtype=dtype, query_lens=query_lens, ctx=ctx, wl=wl, paged=paged, M=M, opts=use_opts))
