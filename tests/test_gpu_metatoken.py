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


@pytest.mark.parametrize("kv_quant", [None, "int8"])
@pytest.mark.parametrize("M", [128, 32])
def test_backend_forward_with_meta_tokens(sb, dev, M, kv_quant):
    """Prompt step with query2 (meta outputs first), chunked second prompt + decodes, then decode
    steps, all with key2/value2; cache contents are those of the plain path. kv_quant="int8": the same
    over Int8KVCache layers (the window keys are what quantize_sym makes of them, the meta rows stay bf16)."""
    from oracle import quant as Q
    bs, wl, nb = 16, 40, 64
    g = torch.Generator().manual_seed(M)
    runner = sb.runner.SwaCacheRunner(1, nb, bs, wl, HKV, D, torch.bfloat16, dev, max_seqs=3, max_chunk_tokens=128,
                                      kv_quant=kv_quant)
    stored = (lambda x: Q.quantize_sym(x, "bf16").astype(np.float32)) if kv_quant else (lambda x: x)
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
            hk = np.concatenate([hk, stored(k[t:t + n].float().numpy())])
            hv = np.concatenate([hv, stored(v[t:t + n].float().numpy())])
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n_split,M", [(1, 128), (4, 128), (3, 100), (4, 1), (2, 33), (5, 200), (0, 128)])
def test_decode_launch_takes_meta_tokens_into_its_softmax(sb, dev, dtype, n_split, M):
    """meta_k/meta_v inside sb_swa_decode: the meta rows' chunks are dealt to the splits of each row's
    window. Against the one-softmax oracle; and against the two-attention form the reference uses
    (window attention, meta attention, log-sum-exp merge) computed by this library's own ops. Rows:
    short, window-saturated, one with an empty window (key_lo past its keys: the meta rows alone);
    with and without the fused append. fp32 queries run the vector kernel, which takes the meta rows the same way
    (tolerance 1e-4 there)."""
    tol = 1e-4 if dtype == torch.float32 else TOL
    bs, wl = 16, 300
    lens = [1, 17, 300, 301, 640, 1000, 33]
    R = len(lens)
    g = torch.Generator().manual_seed(M + n_split)
    nblk = [(L + bs - 1) // bs for L in lens]
    nb = sum(nblk) + 3
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(R, max(nblk), dtype=torch.int32)
    p0 = 0
    for r in range(R):
        tables[r, :nblk[r]] = perm[p0:p0 + nblk[r]]
        p0 += nblk[r]
    kc = torch.randn(nb, bs, HKV, D, generator=g).to(dtype)
    vc = torch.randn(nb, bs, HKV, D, generator=g).to(dtype)
    q = torch.randn(R, HQ, D, generator=g).to(dtype)
    k2 = torch.randn(M, HKV, D, generator=g).to(dtype)
    v2 = torch.randn(M, HKV, D, generator=g).to(dtype)
    key_lo = torch.zeros(R, dtype=torch.int32)
    key_lo[6] = lens[6]                      # nothing of this row's window is visible
    seq = torch.tensor(lens, dtype=torch.int32)

    def keys_of(r, cache):
        rows = [cache[tables[r, i // bs], i % bs] for i in range(lens[r])]
        return torch.stack(rows).float().numpy()

    ref = np.zeros((R, HQ, D))
    for r in range(R):
        k1, v1 = keys_of(r, kc), keys_of(r, vc)
        lo = int(key_lo[r])
        k1, v1 = k1[lo:], v1[lo:]
        if len(k1) == 0:   # a query with no window keys: plain softmax over the meta rows alone
            for h in range(HQ):
                ref[r, h] = A.masked_softmax_attention(q[r:r + 1, h].double().numpy(), k2[:, h // (HQ // HKV)].double().numpy(),
                                                       v2[:, h // (HQ // HKV)].double().numpy(), np.zeros((1, M), bool),
                                                       D ** -0.5)[0]
        else:
            ref[r] = A.metatoken_attention(q[r:r + 1].float().numpy(), None, k1, k2.float().numpy(), v1, v2.float().numpy(),
                                           D ** -0.5, wl + 1)[0]
    args = dict(block_table=tables.to(dev), window_left=wl, key_lo=key_lo.to(dev), n_split=n_split, max_seq_len=max(lens))
    out = sb.ops.swa_decode_attention(q.to(dev), kc.to(dev), vc.to(dev), seq.to(dev), meta_k=k2.to(dev), meta_v=v2.to(dev), **args)
    got = out.float().cpu().numpy()
    assert np.abs(got - ref).max() <= tol
    # the reference's form: two attentions merged by their log-sum-exp
    o1, l1 = sb.ops.swa_decode_attention(q.to(dev), kc.to(dev), vc.to(dev), seq.to(dev), return_lse=True, **args)
    o2, l2 = sb.ops.meta_token_attention(q.to(dev), k2.to(dev), v2.to(dev))
    sb.ops.lse_merge(o1, l1, o2, l2)
    assert np.abs(got - o1.float().cpu().numpy()).max() <= tol
    # the log-sum-exp of the one softmax equals the merged one
    _, lse = sb.ops.swa_decode_attention(q.to(dev), kc.to(dev), vc.to(dev), seq.to(dev), meta_k=k2.to(dev), meta_v=v2.to(dev),
                                         return_lse=True, **args)
    assert torch.allclose(lse, l1, atol=2e-3, rtol=1e-4)


def test_meta_tokens_with_fused_append_and_rejections(sb, dev):
    """Meta rows together with the fused append (bf16 on the matrix cores, fp32 on the vector kernel), and what is refused."""
    bs, wl, M, R = 16, 64, 128, 5
    g = torch.Generator().manual_seed(5)
    lens = [1, 16, 65, 100, 129]
    nblk = [(L + bs - 1) // bs for L in lens]
    nb = sum(nblk)
    tables = torch.zeros(R, max(nblk), dtype=torch.int32)
    p0 = 0
    for r in range(R):
        tables[r, :nblk[r]] = torch.arange(p0, p0 + nblk[r])
        p0 += nblk[r]
    kc = torch.randn(nb, bs, HKV, D, generator=g).bfloat16()
    vc = torch.randn(nb, bs, HKV, D, generator=g).bfloat16()
    q = torch.randn(R, HQ, D, generator=g).bfloat16().to(dev)
    k2 = torch.randn(M, HKV, D, generator=g).bfloat16().to(dev)
    v2 = torch.randn(M, HKV, D, generator=g).bfloat16().to(dev)
    slots = torch.tensor([int(tables[r, (lens[r] - 1) // bs]) * bs + (lens[r] - 1) % bs for r in range(R)])
    newk = torch.stack([kc.view(-1, HKV, D)[s] for s in slots]).to(dev)
    newv = torch.stack([vc.view(-1, HKV, D)[s] for s in slots]).to(dev)
    seq = torch.tensor(lens, dtype=torch.int32, device=dev)
    args = dict(block_table=tables.to(dev), window_left=wl, n_split=2, max_seq_len=max(lens), meta_k=k2, meta_v=v2)
    want = sb.ops.swa_decode_attention(q, kc.to(dev), vc.to(dev), seq, **args)
    # the same step with the newest rows missing from the cache and appended by the launch itself
    kd, vd = kc.clone(), vc.clone()
    kd.view(-1, HKV, D)[slots] = float("nan")
    vd.view(-1, HKV, D)[slots] = float("nan")
    kd, vd = kd.to(dev), vd.to(dev)
    got = sb.ops.swa_decode_attention(q, kd, vd, seq, new_key=newk, new_value=newv, new_slot_mapping=slots.to(dev), **args)
    assert (got.float() - want.float()).abs().max().item() <= TOL
    assert torch.equal(kd.cpu(), kc) and torch.equal(vd.cpu(), vc)
    # fp32 queries (vector kernel): the meta rows go into the same launch there too, the append in front of it
    kf, vf = kc.float(), vc.float()
    kf.view(-1, HKV, D)[slots] = float("nan")
    vf.view(-1, HKV, D)[slots] = float("nan")
    kf, vf = kf.to(dev), vf.to(dev)
    args32 = dict(args, meta_k=k2.float(), meta_v=v2.float())
    got32 = sb.ops.swa_decode_attention(q.float(), kf, vf, seq, new_key=newk.float(), new_value=newv.float(),
                                        new_slot_mapping=slots.to(dev), **args32)
    assert (got32 - want.float()).abs().max().item() <= TOL
    assert torch.equal(kf.cpu(), kc.float()) and torch.equal(vf.cpu(), vc.float())
    with pytest.raises(ValueError):
        sb.ops.swa_decode_attention(q, kc.to(dev), vc.to(dev), seq, block_table=tables.to(dev), window_left=wl,
                                    meta_k=k2[:, :2], meta_v=v2[:, :2])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,wl", [(128, 40), (33, 300), (1, -1), (64, 40)])
def test_many_query_kernel_takes_meta_tokens_into_its_softmax(sb, dev, dtype, M, wl):
    """meta_k/meta_v inside sb_swa_prefill: the meta chunks are walked in front of each tile's window
    chunks. Ragged prompts, some with earlier context (their queries are the last tokens of a longer key
    run); against the one-softmax oracle, and the log-sum-exp against this library's two-attention form."""
    qlens = [5, 64, 100, 257, 1]
    ctx = [0, 30, 0, 200, 77]
    klens = [a + b for a, b in zip(qlens, ctx)]
    g = torch.Generator().manual_seed(M + max(wl, 0))
    Tq, Tk = sum(qlens), sum(klens)
    q = torch.randn(Tq, HQ, D, generator=g).to(dtype)
    k = torch.randn(Tk, HKV, D, generator=g).to(dtype)
    v = torch.randn(Tk, HKV, D, generator=g).to(dtype)
    k2 = torch.randn(M, HKV, D, generator=g).to(dtype)
    v2 = torch.randn(M, HKV, D, generator=g).to(dtype)
    kstart = torch.tensor([sum(klens[:i]) for i in range(len(klens))], dtype=torch.int64)
    args = dict(query_lens=qlens, seq_lens_k=klens, kv_start=kstart.to(dev), window_left=wl)
    out, lse = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), meta_k=k2.to(dev), meta_v=v2.to(dev),
                                            return_lse=True, **args)
    got = out.float().cpu().numpy()
    qo = 0
    for i, (lq, lk) in enumerate(zip(qlens, klens)):
        ks = int(kstart[i])
        ref = A.metatoken_attention(q[qo:qo + lq].float().numpy(), None, k[ks:ks + lk].float().numpy(), k2.float().numpy(),
                                    v[ks:ks + lk].float().numpy(), v2.float().numpy(), D ** -0.5, wl + 1 if wl >= 0 else 0)
        assert np.abs(got[qo:qo + lq] - ref).max() <= TOL, i
        qo += lq
    o1, l1 = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), return_lse=True, **args)
    o2, l2 = sb.ops.meta_token_attention(q.to(dev), k2.to(dev), v2.to(dev))
    sb.ops.lse_merge(o1, l1, o2, l2)
    assert np.abs(got - o1.float().cpu().numpy()).max() <= TOL
    assert torch.allclose(lse, l1, atol=2e-3, rtol=1e-4)
    with pytest.raises(ValueError):
        sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), meta_k=k2.to(dev), **args)


def _byte_code_cache(sb, dev, kind, k, v, slots, nb, bs):
    """K/V rows stored as INT8 codes + per-row scales, or as fp8 codes with tensor scales (0.25, 0.5);
    returns (k cache, v cache, kernel kwargs, rows as the reference's quantise-dequantise leaves them)."""
    from oracle import quant as Q
    Hkv = k.shape[1]
    if kind == "int8":
        kv, sc = sb.ops.alloc_int8_kv_cache(nb, bs, Hkv, D, dev)
        sc.fill_(float("nan"))
        sb.ops.kv_append_int8(k.to(dev), v.to(dev), kv[0], kv[1], sc[0], sc[1], slots.to(dev))
        return kv[0], kv[1], dict(k_scale=sc[0], v_scale=sc[1]), \
            Q.quantize_sym(k.float().numpy(), "bf16"), Q.quantize_sym(v.float().numpy(), "bf16")
    raw = torch.full((2, nb, bs, Hkv, D), 0x7F, dtype=torch.uint8, device=dev)      # unwritten bytes are NaN codes
    kv = raw.view(torch.float8_e4m3fn)
    sb.ops.kv_append_fp8(k.to(dev), v.to(dev), kv[0], kv[1], slots.to(dev), 0.25, 0.5)
    return kv[0], kv[1], dict(fp8_scales=(0.25, 0.5)), \
        Q.fp8_round(k.float().numpy(), 0.25, "bf16"), Q.fp8_round(v.float().numpy(), 0.5, "bf16")


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("n_split,M", [(1, 128), (3, 100), (4, 1), (2, 33), (0, 200)])
def test_decode_over_byte_code_cache_takes_meta_tokens(sb, dev, kind, n_split, M):
    """meta_k/meta_v inside the decode launch over an INT8 / fp8 cache: the meta rows stay bf16 (they are not
    part of the cache) and share the softmax with the dequantised window keys; an fp8 cache's tensor scales,
    folded into the softmax scale and the result, must cancel for them. One-softmax oracle over
    [meta rows | code * scale rounded to bf16]; one row's window is empty (the meta rows alone)."""
    bs, wl = 16, 300
    lens = [1, 17, 300, 301, 640, 1000, 33]
    R = len(lens)
    g = torch.Generator().manual_seed(M + n_split)
    nblk = [(L + bs - 1) // bs for L in lens]
    nb = sum(nblk) + 3
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(R, max(nblk), dtype=torch.int32)
    p0 = 0
    for r in range(R):
        tables[r, :nblk[r]] = perm[p0:p0 + nblk[r]]
        p0 += nblk[r]
    T = sum(lens)
    k = (torch.randn(T, HKV, D, generator=g) * (0.5 + torch.rand(T, HKV, 1, generator=g))).bfloat16()
    v = (torch.randn(T, HKV, D, generator=g) * (1 + torch.rand(T, HKV, 1, generator=g))).bfloat16()
    slots = torch.cat([torch.tensor([int(tables[r, i // bs]) * bs + i % bs for i in range(n)], dtype=torch.int64)
                       for r, n in enumerate(lens)])
    kc, vc, kw, kd, vd = _byte_code_cache(sb, dev, kind, k, v, slots, nb, bs)
    q = torch.randn(R, HQ, D, generator=g).bfloat16()
    k2 = torch.randn(M, HKV, D, generator=g).bfloat16()
    v2 = (torch.randn(M, HKV, D, generator=g) * 2).bfloat16()
    key_lo = torch.zeros(R, dtype=torch.int32)
    key_lo[6] = lens[6]
    ref = np.zeros((R, HQ, D))
    t0 = 0
    for r, n in enumerate(lens):
        k1, v1 = kd[t0 + int(key_lo[r]):t0 + n], vd[t0 + int(key_lo[r]):t0 + n]
        t0 += n
        if len(k1) == 0:
            for h in range(HQ):
                ref[r, h] = A.masked_softmax_attention(q[r:r + 1, h].double().numpy(), k2[:, h // (HQ // HKV)].double().numpy(),
                                                       v2[:, h // (HQ // HKV)].double().numpy(), np.zeros((1, M), bool),
                                                       D ** -0.5)[0]
        else:
            ref[r] = A.metatoken_attention(q[r:r + 1].float().numpy(), None, k1, k2.float().numpy(), v1, v2.float().numpy(),
                                           D ** -0.5, wl + 1)[0]
    args = dict(block_table=tables.to(dev), window_left=wl, key_lo=key_lo.to(dev), n_split=n_split, max_seq_len=max(lens), **kw)
    seq = torch.tensor(lens, dtype=torch.int32, device=dev)
    out, lse = sb.ops.swa_decode_attention(q.to(dev), kc, vc, seq, meta_k=k2.to(dev), meta_v=v2.to(dev), return_lse=True, **args)
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any()
    assert (np.abs(got - ref) <= TOL + 2.0 ** -8 * np.abs(ref)).all()
    # the reference's form over the same cache: two attentions merged by their log-sum-exp
    o1, l1 = sb.ops.swa_decode_attention(q.to(dev), kc, vc, seq, return_lse=True, **args)
    o2, l2 = sb.ops.meta_token_attention(q.to(dev), k2.to(dev), v2.to(dev))
    sb.ops.lse_merge(o1, l1, o2, l2)
    assert (np.abs(got - o1.float().cpu().numpy()) <= TOL + 2.0 ** -8 * np.abs(ref)).all()
    assert torch.allclose(lse, l1, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("M,wl", [(128, 40), (33, 300), (1, -1), (70, 70)])
def test_many_query_kernel_over_byte_code_cache_takes_meta_tokens(sb, dev, kind, M, wl):
    """meta_k/meta_v inside the many-query launch reading an INT8 / fp8 paged cache (chunked prefill): the
    meta chunks go through the kernel's LDS stage as elements ahead of the dequantised window chunks."""
    bs = 16
    qlens, klens = [40, 5, 130, 1], [100, 5, 230, 64]
    g = torch.Generator().manual_seed(M + max(wl, 0))
    need = [(n + bs - 1) // bs for n in klens]
    nb = sum(need) + 2
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(len(klens), max(need), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
    Tk, Tq = sum(klens), sum(qlens)
    k = (torch.randn(Tk, HKV, D, generator=g) * (0.5 + torch.rand(Tk, HKV, 1, generator=g))).bfloat16()
    v = (torch.randn(Tk, HKV, D, generator=g) * (1 + torch.rand(Tk, HKV, 1, generator=g))).bfloat16()
    q = torch.randn(Tq, HQ, D, generator=g).bfloat16()
    k2 = torch.randn(M, HKV, D, generator=g).bfloat16()
    v2 = (torch.randn(M, HKV, D, generator=g) * 2).bfloat16()
    slots = torch.cat([torch.tensor([int(tables[b, i // bs]) * bs + i % bs for i in range(n)], dtype=torch.int64)
                       for b, n in enumerate(klens)])
    kc, vc, kw, kd, vd = _byte_code_cache(sb, dev, kind, k, v, slots, nb, bs)
    args = dict(query_lens=qlens, seq_lens_k=klens, block_table=tables.to(dev), window_left=wl, return_lse=True, **kw)
    out, lse = sb.ops.swa_prefill_attention(q.to(dev), kc, vc, meta_k=k2.to(dev), meta_v=v2.to(dev), **args)
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any() and not torch.isnan(lse).any()
    qo = ko = 0
    for i, (lq, lk) in enumerate(zip(qlens, klens)):
        ref = A.metatoken_attention(q[qo:qo + lq].float().numpy(), None, kd[ko:ko + lk], k2.float().numpy(),
                                    vd[ko:ko + lk], v2.float().numpy(), D ** -0.5, wl + 1 if wl >= 0 else 0)
        assert (np.abs(got[qo:qo + lq] - ref) <= TOL + 2.0 ** -8 * np.abs(ref)).all(), i
        qo += lq
        ko += lk
    o1, l1 = sb.ops.swa_prefill_attention(q.to(dev), kc, vc, **args)
    o2, l2 = sb.ops.meta_token_attention(q.to(dev), k2.to(dev), v2.to(dev))
    sb.ops.lse_merge(o1, l1, o2, l2)
    assert (np.abs(got - o1.float().cpu().numpy()) <= TOL + 2.0 ** -7 * np.abs(got)).all()
    assert torch.allclose(lse, l1, atol=2e-3, rtol=1e-4)
