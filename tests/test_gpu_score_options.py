"""Soft cap and ALiBi slopes on the attention scores (also together with meta tokens, and in the fp32 vector
kernel): the two options the backend hands to every flash-attn call
(vllm_hymeta/attention/meta_attention.py:665-690, :758-759, :882-883, :916-918, :950-952, :978-980), in the
decode kernels (element, INT8 and fp8 caches; fixed and balanced split), the many-query kernel (in-flight and
paged keys) and through MetaAttentionImpl.forward, against the float64 oracle.
Tolerance: max-abs 2e-2 (bf16), 5e-3 (fp16), 1e-4 (fp32), against fp64 mathematics on the same (for byte-code
caches: dequantised) rows."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle import quant as Q

pytestmark = pytest.mark.gpu

D = 128
TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3, torch.float32: 1e-4}
OPTIONS = [dict(softcap=0.0, alibi=True), dict(softcap=3.0, alibi=False), dict(softcap=1.5, alibi=True)]


def slopes_for(Hq):
    return [2.0 ** (-8.0 * (h + 1) / Hq) for h in range(Hq)]           # the usual geometric ALiBi slopes


def paged_problem(lens, bs, Hkv, dtype, seed, slack=4):
    g = torch.Generator().manual_seed(seed)
    need = [(n + bs - 1) // bs for n in lens]
    nb = sum(need) + slack
    perm = torch.randperm(nb, generator=g)
    kv = torch.randn(2, nb, bs, Hkv, D, generator=g).to(dtype)
    tables = torch.zeros(len(lens), max(need), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
    return kv, tables


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hq,Hkv", [(28, 4), (8, 2), (5, 1)])
@pytest.mark.parametrize("opt", OPTIONS)
@pytest.mark.parametrize("wl,n_split,balanced", [(64, 1, False), (100, 3, False), (-1, 2, False), (80, 2, True)])
def test_decode_with_soft_cap_and_alibi(sb, dev, dtype, Hq, Hkv, opt, wl, n_split, balanced):
    bs = 16
    lens = [1, 16, 17, 65, 129, 300]
    kv, tables = paged_problem(lens, bs, Hkv, dtype, seed=Hq + n_split)
    q = (2.0 * torch.randn(len(lens), Hq, D, generator=torch.Generator().manual_seed(3))).to(dtype)  # scores large enough for the cap to bite
    slopes = slopes_for(Hq) if opt["alibi"] else None
    scale = D ** -0.5
    out, lse = sb.ops.swa_decode_attention(
        q.to(dev), kv[0].to(dev), kv[1].to(dev), torch.tensor(lens, dtype=torch.int32, device=dev),
        block_table=tables.to(dev), window_left=wl, scale=scale, n_split=n_split, balanced=balanced, return_lse=True,
        softcap=opt["softcap"], alibi_slopes=None if slopes is None else torch.tensor(slopes, device=dev))
    ref, ref_lse = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(),
                                            lens, scale, wl, return_lse=True, softcap=opt["softcap"], alibi_slopes=slopes)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= TOL[dtype]
    assert np.abs(lse.cpu().numpy() - ref_lse).max() <= 2e-3
    plain = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(),
                                     lens, scale, wl)
    assert np.abs(plain - ref).max() > 5 * TOL[dtype]                   # the options do change the result here


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("opt", OPTIONS)
def test_decode_over_byte_code_cache_with_soft_cap_and_alibi(sb, dev, kind, opt):
    Hq, Hkv, bs, wl = 28, 4, 16, 150
    lens = [1, 33, 150, 151, 400]
    g = torch.Generator().manual_seed(5)
    nblk = [(n + bs - 1) // bs for n in lens]
    nb = sum(nblk) + 2
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(len(lens), max(nblk), dtype=torch.int32)
    p0 = 0
    for r, n in enumerate(nblk):
        tables[r, :n] = perm[p0:p0 + n]; p0 += n
    T = sum(lens)
    k = (torch.randn(T, Hkv, D, generator=g) * (0.5 + torch.rand(T, Hkv, 1, generator=g))).bfloat16()
    v = torch.randn(T, Hkv, D, generator=g).bfloat16()
    slots = torch.cat([torch.tensor([int(tables[r, i // bs]) * bs + i % bs for i in range(n)], dtype=torch.int64)
                       for r, n in enumerate(lens)])
    if kind == "int8":
        kvc, sc = sb.ops.alloc_int8_kv_cache(nb, bs, Hkv, D, dev)
        sb.ops.kv_append_int8(k.to(dev), v.to(dev), kvc[0], kvc[1], sc[0], sc[1], slots.to(dev))
        kw = dict(k_scale=sc[0], v_scale=sc[1])
        kd, vd = Q.quantize_sym(k.float().numpy(), "bf16"), Q.quantize_sym(v.float().numpy(), "bf16")
    else:
        kvc = torch.zeros(2, nb, bs, Hkv, D, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        sb.ops.kv_append_fp8(k.to(dev), v.to(dev), kvc[0], kvc[1], slots.to(dev), 0.25, 0.5)
        kw = dict(fp8_scales=(0.25, 0.5))
        kd, vd = Q.fp8_round(k.float().numpy(), 0.25, "bf16"), Q.fp8_round(v.float().numpy(), 0.5, "bf16")
    q = (2.0 * torch.randn(len(lens), Hq, D, generator=g)).bfloat16()
    slopes = slopes_for(Hq) if opt["alibi"] else None
    out = sb.ops.swa_decode_attention(
        q.to(dev), kvc[0], kvc[1], torch.tensor(lens, dtype=torch.int32, device=dev), block_table=tables.to(dev),
        window_left=wl, scale=D ** -0.5, n_split=2, softcap=opt["softcap"],
        alibi_slopes=None if slopes is None else torch.tensor(slopes, device=dev), **kw)
    # the oracle attends to the dequantised rows, laid out as one block per sequence
    off = np.cumsum([0] + lens)
    for r, n in enumerate(lens):
        ref = A.paged_decode_attention(q[r:r + 1].float().numpy(), kd[off[r]:off[r + 1]][None], vd[off[r]:off[r + 1]][None],
                                       np.zeros((1, 1), np.int32), [n], D ** -0.5, wl, softcap=opt["softcap"], alibi_slopes=slopes)
        assert np.abs(out[r].float().cpu().numpy() - ref[0]).max() <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hq,Hkv", [(28, 4), (6, 2), (5, 1)])
@pytest.mark.parametrize("opt", OPTIONS)
@pytest.mark.parametrize("paged", [False, True])
def test_many_query_kernel_with_soft_cap_and_alibi(sb, dev, dtype, Hq, Hkv, opt, paged):
    """Prompts and chunked prefill: query j of a sequence sits at key position Lk - Lq + j."""
    wl, bs = 70, 16
    query_lens = [1, 17, 64, 130] if not paged else [40, 3, 130, 1]
    ctx = [0, 0, 0, 0] if not paged else [60, 0, 200, 33]
    lens_k = [a + b for a, b in zip(query_lens, ctx)]
    g = torch.Generator().manual_seed(Hq + (7 if paged else 0))
    cu_q = np.cumsum([0] + query_lens); cu_k = np.cumsum([0] + lens_k)
    q = (2.0 * torch.randn(int(cu_q[-1]), Hq, D, generator=g)).to(dtype)
    k = torch.randn(int(cu_k[-1]), Hkv, D, generator=g).to(dtype)
    v = torch.randn(int(cu_k[-1]), Hkv, D, generator=g).to(dtype)
    slopes = slopes_for(Hq) if opt["alibi"] else None
    kw = dict(softcap=opt["softcap"], alibi_slopes=None if slopes is None else torch.tensor(slopes, device=dev))
    if paged:
        need = [(n + bs - 1) // bs for n in lens_k]
        nb = sum(need) + 3
        perm = torch.randperm(nb, generator=g)
        kc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype); vc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype)
        tables = torch.zeros(len(lens_k), max(need), dtype=torch.int32)
        p = 0
        for s, n in enumerate(need):
            tables[s, :n] = perm[p:p + n]; p += n
            for i in range(lens_k[s]):
                kc[int(tables[s, i // bs]), i % bs] = k[cu_k[s] + i]
                vc[int(tables[s, i // bs]), i % bs] = v[cu_k[s] + i]
        out = sb.ops.swa_prefill_attention(q.to(dev), kc.to(dev), vc.to(dev), query_lens=query_lens, seq_lens_k=lens_k,
                                           block_table=tables.to(dev), window_left=wl, scale=D ** -0.5, **kw)
    else:
        out = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=query_lens, window_left=wl,
                                           scale=D ** -0.5, **kw)
    ref = A.varlen_window_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), cu_q, cu_k, D ** -0.5, wl,
                                    softcap=opt["softcap"], alibi_slopes=slopes)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= TOL[dtype]
    plain = A.varlen_window_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), cu_q, cu_k, D ** -0.5, wl)
    assert np.abs(plain - ref).max() > 5 * TOL[dtype]


def test_backend_passes_the_options_on(sb, dev):
    """MetaAttentionImpl(alibi_slopes=..., logits_soft_cap=...): a prompt step over the in-flight keys, then
    decode steps through the paged cache, against the oracle with the same options."""
    Hq, Hkv, bs, wl, nb = 28, 4, 16, 40, 32
    slopes = slopes_for(Hq)
    impl = sb.MetaAttentionImpl(Hq, D, D ** -0.5, Hkv, slopes, wl + 1, "auto", logits_soft_cap=2.5)
    assert impl.logits_soft_cap == 2.5 and impl.alibi_slopes.shape == (Hq,)
    runner = sb.runner.SwaCacheRunner(1, nb, bs, wl, Hkv, D, torch.bfloat16, dev, max_seqs=2, max_chunk_tokens=128)
    g = torch.Generator().manual_seed(1)
    hist_k = {0: [], 1: []}; hist_v = {0: [], 1: []}
    for sid in (0, 1):
        runner.add_seq(sid)

    def step(prompts, decodes):
        T = sum(n for _, n in prompts) + len(decodes)
        q = (2.0 * torch.randn(T, Hq, D, generator=g)).bfloat16()
        k = torch.randn(T, Hkv, D, generator=g).bfloat16(); v = torch.randn(T, Hkv, D, generator=g).bfloat16()
        meta = runner.build_step(prompts, decodes)
        out = torch.empty(T, Hq, D, dtype=torch.bfloat16, device=dev)
        impl.forward(None, q.to(dev), k.to(dev), v.to(dev), None, None, None, runner.kv_caches[0], meta, output=out)
        t = 0
        for sid, n in prompts + [(d, 1) for d in decodes]:
            hist_k[sid] += list(k[t:t + n].float().numpy()); hist_v[sid] += list(v[t:t + n].float().numpy())
            L = len(hist_k[sid])
            ref = A.varlen_window_attention(q[t:t + n].float().numpy(), np.stack(hist_k[sid]), np.stack(hist_v[sid]),
                                            [0, n], [0, L], D ** -0.5, wl, softcap=2.5, alibi_slopes=slopes)
            assert np.abs(out[t:t + n].float().cpu().numpy() - ref).max() <= 2e-2
            t += n

    step([(0, 30), (1, 75)], [])
    for _ in range(20):
        step([], [0, 1])
    with pytest.raises(ValueError, match="one slope per query head"):
        sb.MetaAttentionImpl(Hq, D, 1.0, Hkv, [0.5] * 3, wl + 1, "auto")
    with pytest.raises(ValueError, match="logits_soft_cap"):
        sb.MetaAttentionImpl(Hq, D, 1.0, Hkv, None, wl + 1, "auto", logits_soft_cap=-1.0)


@pytest.mark.parametrize("dtype,force_valu,G", [(torch.float32, False, 7), (torch.float32, False, 1), (torch.bfloat16, True, 7),
                                                (torch.float16, True, 4)])
@pytest.mark.parametrize("opt", OPTIONS)
def test_vector_kernel_with_soft_cap_and_alibi(sb, dev, dtype, force_valu, G, opt):
    """fp32 queries (and bf16/fp16 forced onto the vector ALUs): the same two options in the vector kernel."""
    Hkv, bs, wl = 2, 16, 90
    Hq = Hkv * G
    lens = [1, 16, 17, 65, 129, 300]
    kv, tables = paged_problem(lens, bs, Hkv, dtype, seed=G)
    q = (2.0 * torch.randn(len(lens), Hq, D, generator=torch.Generator().manual_seed(4))).to(dtype)
    slopes = slopes_for(Hq) if opt["alibi"] else None
    out, lse = sb.ops.swa_decode_attention(
        q.to(dev), kv[0].to(dev), kv[1].to(dev), torch.tensor(lens, dtype=torch.int32, device=dev),
        block_table=tables.to(dev), window_left=wl, scale=D ** -0.5, n_split=2, return_lse=True, force_valu=force_valu,
        softcap=opt["softcap"], alibi_slopes=None if slopes is None else torch.tensor(slopes, device=dev))
    ref, ref_lse = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(),
                                            lens, D ** -0.5, wl, return_lse=True, softcap=opt["softcap"], alibi_slopes=slopes)
    tol = 1e-5 if dtype == torch.float32 else TOL[dtype]
    assert np.abs(out.float().cpu().numpy() - ref).max() <= tol
    assert np.abs(lse.cpu().numpy() - ref_lse).max() <= 2e-3
    plain = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(),
                                     lens, D ** -0.5, wl)
    assert np.abs(plain - ref).max() > 5 * 2e-2


def _gather(kv, tables, b, n, bs):
    return (np.stack([kv[0][int(tables[b, i // bs]), i % bs].float().numpy() for i in range(n)]) if n else np.zeros((0,) + tuple(kv.shape[3:])),
            np.stack([kv[1][int(tables[b, i // bs]), i % bs].float().numpy() for i in range(n)]) if n else np.zeros((0,) + tuple(kv.shape[3:])))


@pytest.mark.parametrize("dtype,force_valu", [(torch.bfloat16, False), (torch.float16, False), (torch.float32, False),
                                              (torch.bfloat16, True)])
@pytest.mark.parametrize("opt", OPTIONS + [dict(softcap=0.0, alibi=False)])
@pytest.mark.parametrize("M,n_split,stack", [(1, 1, None), (40, 3, None), (100, 2, (7, 50))])
def test_decode_with_meta_rows_and_options(sb, dev, dtype, force_valu, opt, M, n_split, stack):
    """Meta rows inside the decode launch together with the score options: the cap on their scores, and the
    ALiBi term of the reference's stacked second attention, -slope |row0 + r + M - rows - j| (fa_kernel_metatoken.py:
    169-188), against the one-softmax oracle; on the matrix-core kernel and on the vector kernel (fp32 queries, or
    forced)."""
    Hq, Hkv, bs, wl = 28, 4, 16, 70
    lens = [1, 17, 0, 65, 129, 300]
    R = len(lens)
    kv, tables = paged_problem([max(n, 1) for n in lens], bs, Hkv, dtype, seed=M)
    g = torch.Generator().manual_seed(9)
    q = (2.0 * torch.randn(R, Hq, D, generator=g)).to(dtype)
    k2 = torch.randn(M, Hkv, D, generator=g).to(dtype); v2 = torch.randn(M, Hkv, D, generator=g).to(dtype)
    slopes = slopes_for(Hq) if opt["alibi"] else None
    kw = {} if stack is None else dict(meta_bias=stack)
    out = sb.ops.swa_decode_attention(
        q.to(dev), kv[0].to(dev), kv[1].to(dev), torch.tensor(lens, dtype=torch.int32, device=dev),
        block_table=tables.to(dev), window_left=wl, scale=D ** -0.5, n_split=n_split, balanced=False,
        meta_k=k2.to(dev), meta_v=v2.to(dev), softcap=opt["softcap"], force_valu=force_valu,
        alibi_slopes=None if slopes is None else torch.tensor(slopes, device=dev), **kw).float().cpu().numpy()
    row0, rows = stack if stack else (0, R)
    for r, n in enumerate(lens):
        k1, v1 = _gather(kv, tables, r, n, bs)
        ref = A.metatoken_attention(q[r:r + 1].float().numpy(), None, k1, k2.float().numpy(), v1, v2.float().numpy(), D ** -0.5,
                                    wl + 1, softcap=opt["softcap"], alibi_slopes=slopes, stack_row0=row0 + r, stack_rows=rows)
        assert np.abs(out[r] - ref[0]).max() <= TOL[dtype], (r, n)


@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_decode_over_byte_code_cache_with_meta_rows_and_options(sb, dev, kind):
    Hq, Hkv, bs, wl, M = 28, 4, 16, 150, 37
    lens = [1, 33, 150, 151, 400]
    g = torch.Generator().manual_seed(6)
    nblk = [(n + bs - 1) // bs for n in lens]
    nb = sum(nblk) + 2
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(len(lens), max(nblk), dtype=torch.int32)
    p0 = 0
    for r, n in enumerate(nblk):
        tables[r, :n] = perm[p0:p0 + n]; p0 += n
    T = sum(lens)
    k = torch.randn(T, Hkv, D, generator=g).bfloat16(); v = torch.randn(T, Hkv, D, generator=g).bfloat16()
    slots = torch.cat([torch.tensor([int(tables[r, i // bs]) * bs + i % bs for i in range(n)], dtype=torch.int64)
                       for r, n in enumerate(lens)])
    if kind == "int8":
        kvc, sc = sb.ops.alloc_int8_kv_cache(nb, bs, Hkv, D, dev)
        sb.ops.kv_append_int8(k.to(dev), v.to(dev), kvc[0], kvc[1], sc[0], sc[1], slots.to(dev))
        kw = dict(k_scale=sc[0], v_scale=sc[1])
        kd, vd = Q.quantize_sym(k.float().numpy(), "bf16"), Q.quantize_sym(v.float().numpy(), "bf16")
    else:
        kvc = torch.zeros(2, nb, bs, Hkv, D, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        sb.ops.kv_append_fp8(k.to(dev), v.to(dev), kvc[0], kvc[1], slots.to(dev), 0.25, 0.5)
        kw = dict(fp8_scales=(0.25, 0.5))
        kd, vd = Q.fp8_round(k.float().numpy(), 0.25, "bf16"), Q.fp8_round(v.float().numpy(), 0.5, "bf16")
    q = (2.0 * torch.randn(len(lens), Hq, D, generator=g)).bfloat16()
    k2 = torch.randn(M, Hkv, D, generator=g).bfloat16(); v2 = torch.randn(M, Hkv, D, generator=g).bfloat16()
    slopes = slopes_for(Hq)
    out = sb.ops.swa_decode_attention(
        q.to(dev), kvc[0], kvc[1], torch.tensor(lens, dtype=torch.int32, device=dev), block_table=tables.to(dev),
        window_left=wl, scale=D ** -0.5, n_split=2, softcap=1.5, alibi_slopes=torch.tensor(slopes, device=dev),
        meta_k=k2.to(dev), meta_v=v2.to(dev), **kw).float().cpu().numpy()
    off = np.cumsum([0] + lens)
    for r, n in enumerate(lens):
        ref = A.metatoken_attention(q[r:r + 1].float().numpy(), None, kd[off[r]:off[r + 1]], k2.float().numpy(),
                                    vd[off[r]:off[r + 1]], v2.float().numpy(), D ** -0.5, wl + 1, softcap=1.5,
                                    alibi_slopes=slopes, stack_row0=r, stack_rows=len(lens))
        assert np.abs(out[r] - ref[0]).max() <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("opt", OPTIONS)
@pytest.mark.parametrize("paged", [False, True])
def test_many_query_kernel_with_meta_rows_and_options(sb, dev, dtype, opt, paged):
    """Prompts / chunked prompts with meta rows and the score options: the stacked rows of the second attention
    are the packed query rows (fa_kernel_metatoken.py:258-275)."""
    Hq, Hkv, wl, bs, M = 28, 4, 70, 16, 45
    query_lens = [1, 17, 64, 130] if not paged else [40, 3, 130, 1]
    ctx = [0, 0, 0, 0] if not paged else [60, 0, 200, 33]
    lens_k = [a + b for a, b in zip(query_lens, ctx)]
    g = torch.Generator().manual_seed(11 + (7 if paged else 0))
    cu_q = np.cumsum([0] + query_lens); cu_k = np.cumsum([0] + lens_k)
    q = (2.0 * torch.randn(int(cu_q[-1]), Hq, D, generator=g)).to(dtype)
    k = torch.randn(int(cu_k[-1]), Hkv, D, generator=g).to(dtype)
    v = torch.randn(int(cu_k[-1]), Hkv, D, generator=g).to(dtype)
    k2 = torch.randn(M, Hkv, D, generator=g).to(dtype); v2 = torch.randn(M, Hkv, D, generator=g).to(dtype)
    slopes = slopes_for(Hq) if opt["alibi"] else None
    N = int(cu_q[-1]) + M                                      # the meta tokens' own queries close the stacked sequence
    kw = dict(softcap=opt["softcap"], alibi_slopes=None if slopes is None else torch.tensor(slopes, device=dev),
              meta_k=k2.to(dev), meta_v=v2.to(dev), meta_bias=(0, N))
    if paged:
        need = [(n + bs - 1) // bs for n in lens_k]
        nb = sum(need) + 3
        perm = torch.randperm(nb, generator=g)
        kc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype); vc = torch.randn(nb, bs, Hkv, D, generator=g).to(dtype)
        tables = torch.zeros(len(lens_k), max(need), dtype=torch.int32)
        p = 0
        for s_, n in enumerate(need):
            tables[s_, :n] = perm[p:p + n]; p += n
            for i in range(lens_k[s_]):
                kc[int(tables[s_, i // bs]), i % bs] = k[cu_k[s_] + i]
                vc[int(tables[s_, i // bs]), i % bs] = v[cu_k[s_] + i]
        out = sb.ops.swa_prefill_attention(q.to(dev), kc.to(dev), vc.to(dev), query_lens=query_lens, seq_lens_k=lens_k,
                                           block_table=tables.to(dev), window_left=wl, scale=D ** -0.5, **kw)
    else:
        out = sb.ops.swa_prefill_attention(q.to(dev), k.to(dev), v.to(dev), query_lens=query_lens, window_left=wl,
                                           scale=D ** -0.5, **kw)
    out = out.float().cpu().numpy()
    for s_ in range(len(query_lens)):
        qs, ks = slice(cu_q[s_], cu_q[s_ + 1]), slice(cu_k[s_], cu_k[s_ + 1])
        ref = A.metatoken_attention(q[qs].float().numpy(), None, k[ks].float().numpy(), k2.float().numpy(), v[ks].float().numpy(),
                                    v2.float().numpy(), D ** -0.5, wl + 1, softcap=opt["softcap"], alibi_slopes=slopes,
                                    stack_row0=int(cu_q[s_]), stack_rows=N)
        assert np.abs(out[qs] - ref).max() <= TOL[dtype], s_


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_backend_with_meta_tokens_and_options(sb, dev, dtype):
    """MetaAttentionImpl.forward with key2/value2/query2 AND logits_soft_cap / alibi_slopes: a prompt step (meta
    queries in front of the output), then decode steps, against the oracle's stacked-sequence convention. fp32
    queries take every piece of the step through the vector kernel."""
    Hq, Hkv, bs, wl, nb, M = 28, 4, 16, 40, 32, 12
    slopes = slopes_for(Hq)
    impl = sb.MetaAttentionImpl(Hq, D, D ** -0.5, Hkv, slopes, wl + 1, "auto", logits_soft_cap=2.5, num_meta_tokens=M)
    runner = sb.runner.SwaCacheRunner(1, nb, bs, wl, Hkv, D, dtype, dev, max_seqs=2, max_chunk_tokens=128)
    g = torch.Generator().manual_seed(2)
    k2 = torch.randn(M, Hkv, D, generator=g).to(dtype); v2 = torch.randn(M, Hkv, D, generator=g).to(dtype)
    q2 = (2.0 * torch.randn(M, Hq, D, generator=g)).to(dtype)
    hist_k = {0: [], 1: []}; hist_v = {0: [], 1: []}
    for sid in (0, 1):
        runner.add_seq(sid)

    def step(prompts, decodes):
        T = sum(n for _, n in prompts) + len(decodes)
        q = (2.0 * torch.randn(T, Hq, D, generator=g)).to(dtype)
        k = torch.randn(T, Hkv, D, generator=g).to(dtype); v = torch.randn(T, Hkv, D, generator=g).to(dtype)
        meta = runner.build_step(prompts, decodes)
        with_q2 = bool(prompts)
        out = torch.empty(T + (M if with_q2 else 0), Hq, D, dtype=dtype, device=dev)
        impl.forward(None, q.to(dev), k.to(dev), v.to(dev), q2.to(dev) if with_q2 else None, k2.to(dev), v2.to(dev),
                     runner.kv_caches[0], meta, output=out)
        o = out.float().cpu().numpy()
        n_prompt = sum(n for _, n in prompts)
        base = M if with_q2 else 0
        t = 0
        first = True
        for sid, n in prompts:
            hist_k[sid] += list(k[t:t + n].float().numpy()); hist_v[sid] += list(v[t:t + n].float().numpy())
            ref = A.metatoken_attention(q[t:t + n].float().numpy(), q2.float().numpy() if first else None, np.stack(hist_k[sid]),
                                        k2.float().numpy(), np.stack(hist_v[sid]), v2.float().numpy(), D ** -0.5, wl + 1,
                                        softcap=2.5, alibi_slopes=slopes, stack_row0=t, stack_rows=n_prompt + M)
            assert np.abs(o[base + t:base + t + n] - ref[:n]).max() <= TOL[dtype]
            if first:
                assert np.abs(o[:M] - ref[n:]).max() <= TOL[dtype]       # the meta tokens' own outputs come first
            first = False
            t += n
        for i, sid in enumerate(decodes):
            hist_k[sid] += list(k[t:t + 1].float().numpy()); hist_v[sid] += list(v[t:t + 1].float().numpy())
            ref = A.metatoken_attention(q[t:t + 1].float().numpy(), None, np.stack(hist_k[sid]), k2.float().numpy(),
                                        np.stack(hist_v[sid]), v2.float().numpy(), D ** -0.5, wl + 1, softcap=2.5,
                                        alibi_slopes=slopes, stack_row0=i, stack_rows=len(decodes))
            assert np.abs(o[base + t] - ref[0]).max() <= TOL[dtype]
            t += 1

    step([(0, 30), (1, 75)], [])
    for _ in range(6):
        step([], [0, 1])
