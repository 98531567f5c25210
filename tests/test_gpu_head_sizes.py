"""Head sizes other than 128: the backend's list is the reference's (32 .. 256 in steps of 32,
vllm_hymeta/attention/meta_attention.py:57-59). The matrix-core kernels are built for 128; the other sizes run
every piece of a step on the vector kernel (8, 16 or 32 lanes per key row). Likewise any GQA group size: the
vector kernel cuts a group it is not built for into parts. Against the float64 oracle.
Tolerance: max-abs 2e-2 (bf16), 5e-3 (fp16), 1e-5 (fp32; 1e-4 with soft cap / ALiBi)."""
import numpy as np
import pytest
import torch

from oracle import attention as A

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3, torch.float32: 1e-5}
SIZES = [32, 64, 96, 160, 192, 224, 256]


def paged_problem(lens, bs, Hkv, D, dtype, seed, slack=3):
    g = torch.Generator().manual_seed(seed)
    need = [(max(n, 1) + bs - 1) // bs for n in lens]
    nb = sum(need) + slack
    perm = torch.randperm(nb, generator=g)
    kv = torch.randn(2, nb, bs, Hkv, D, generator=g).to(dtype)
    tables = torch.zeros(len(lens), max(need), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
    return kv, tables


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D", SIZES)
@pytest.mark.parametrize("Hq,Hkv,wl,n_split", [(28, 4, 64, 1), (8, 2, 37, 3), (8, 8, -1, 2), (4, 1, 100, 0)])
def test_paged_decode_vs_oracle(sb, dev, dtype, D, Hq, Hkv, wl, n_split):
    bs = 16
    lens = [1, 15, 16, 17, 64, 65, 129, 200]
    kv, tables = paged_problem(lens, bs, Hkv, D, dtype, seed=D + Hq)
    q = torch.randn(len(lens), Hq, D, generator=torch.Generator().manual_seed(2)).to(dtype)
    scale = D ** -0.5
    out, lse = sb.ops.swa_decode_attention(q.to(dev), kv[0].to(dev), kv[1].to(dev), torch.tensor(lens, dtype=torch.int32, device=dev),
                                           block_table=tables.to(dev), window_left=wl, scale=scale, n_split=n_split,
                                           return_lse=True)
    ref, ref_lse = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(),
                                            lens, scale, wl, return_lse=True)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= TOL[dtype]
    assert np.abs(lse.cpu().numpy() - ref_lse).max() <= 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("D", [64, 96, 256])
def test_decode_with_fused_append_meta_rows_and_options(sb, dev, dtype, D):
    """Everything the launch can carry, at once: the step's newest K/V rows (appended by the call), meta rows,
    soft cap and ALiBi; one row with an empty window."""
    Hq, Hkv, bs, wl, M = 8, 2, 16, 70, 37
    lens = [1, 17, 0, 65, 129, 300]
    R = len(lens)
    kv, tables = paged_problem(lens, bs, Hkv, D, dtype, seed=D)
    g = torch.Generator().manual_seed(9)
    q = (2.0 * torch.randn(R, Hq, D, generator=g)).to(dtype)
    k2 = torch.randn(M, Hkv, D, generator=g).to(dtype); v2 = torch.randn(M, Hkv, D, generator=g).to(dtype)
    slopes = [2.0 ** (-8.0 * (h + 1) / Hq) for h in range(Hq)]
    # the newest row of every sequence leaves the cache (NaN there) and comes with the call instead
    rows = [r for r in range(R) if lens[r] > 0]
    slots = torch.full((R,), -1, dtype=torch.int64)
    newk = torch.zeros(R, Hkv, D, dtype=dtype); newv = torch.zeros(R, Hkv, D, dtype=dtype)
    want = kv.clone()
    holed = kv.clone()
    for r in rows:
        i = lens[r] - 1
        blk, off = int(tables[r, i // bs]), i % bs
        slots[r] = blk * bs + off
        newk[r], newv[r] = kv[0, blk, off], kv[1, blk, off]
        holed[:, blk, off] = float("nan")
    kd, vd = holed[0].to(dev), holed[1].to(dev)
    out = sb.ops.swa_decode_attention(
        q.to(dev), kd, vd, torch.tensor(lens, dtype=torch.int32, device=dev), block_table=tables.to(dev), window_left=wl,
        scale=D ** -0.5, n_split=2, new_key=newk.to(dev), new_value=newv.to(dev), new_slot_mapping=slots.to(dev),
        meta_k=k2.to(dev), meta_v=v2.to(dev), softcap=2.5, alibi_slopes=torch.tensor(slopes, device=dev)).float().cpu().numpy()
    assert torch.equal(kd.cpu(), want[0]) and torch.equal(vd.cpu(), want[1])
    tol = 1e-4 if dtype == torch.float32 else TOL[dtype]
    for r, n in enumerate(lens):
        k1 = np.stack([want[0, int(tables[r, i // bs]), i % bs].float().numpy() for i in range(n)]) if n else np.zeros((0, Hkv, D), np.float32)
        v1 = np.stack([want[1, int(tables[r, i // bs]), i % bs].float().numpy() for i in range(n)]) if n else np.zeros((0, Hkv, D), np.float32)
        ref = A.metatoken_attention(q[r:r + 1].float().numpy(), None, k1, k2.float().numpy(), v1, v2.float().numpy(), D ** -0.5,
                                    wl + 1, softcap=2.5, alibi_slopes=slopes, stack_row0=r, stack_rows=R)
        assert np.abs(out[r] - ref[0]).max() <= tol, (r, n)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("D", [64, 256])
def test_backend_forward_at_other_head_sizes(sb, dev, dtype, D):
    """MetaAttentionImpl.forward with head_size 64 / 256: plain prompts, a chunked prompt next to decodes, decode
    steps (fused append), through the block manager; outputs against the oracle over each sequence's own history,
    cache contents against the rows that were appended."""
    Hq, Hkv, bs, wl, nb = 8, 2, 16, 40, 40
    assert D in sb.MetaAttentionBackend.get_supported_head_sizes()
    impl = sb.MetaAttentionImpl(Hq, D, D ** -0.5, Hkv, None, wl + 1, "auto")
    runner = sb.runner.SwaCacheRunner(1, nb, bs, wl, Hkv, D, dtype, dev, max_seqs=3, max_chunk_tokens=128)
    g = torch.Generator().manual_seed(D)
    hist_k = {s: [] for s in range(3)}; hist_v = {s: [] for s in range(3)}
    for sid in range(3):
        runner.add_seq(sid)

    def step(prompts, decodes, chunked=False):
        T = sum(n for _, n in prompts) + len(decodes)
        q = torch.randn(T, Hq, D, generator=g).to(dtype)
        k = torch.randn(T, Hkv, D, generator=g).to(dtype); v = torch.randn(T, Hkv, D, generator=g).to(dtype)
        meta = runner.build_step(prompts, decodes, chunked_prefill=chunked)
        out = torch.full((T, Hq, D), float("nan"), dtype=dtype, device=dev)
        impl.forward(None, q.to(dev), k.to(dev), v.to(dev), None, None, None, runner.kv_caches[0], meta, output=out)
        got = out.float().cpu().numpy()
        t = 0
        for sid, n in list(prompts) + [(s, 1) for s in decodes]:
            hist_k[sid] += list(k[t:t + n].float().numpy()); hist_v[sid] += list(v[t:t + n].float().numpy())
            L = len(hist_k[sid])
            ref = A.varlen_window_attention(q[t:t + n].float().numpy(), np.stack(hist_k[sid]), np.stack(hist_v[sid]),
                                            [0, n], [0, L], D ** -0.5, wl)
            assert np.abs(got[t:t + n] - ref).max() <= TOL[dtype], (sid, n)
            t += n

    step([(0, 30), (1, 75)], [])
    step([(2, 50)], [0, 1], chunked=True)
    for _ in range(bs + 2):
        step([], [0, 1, 2])


@pytest.mark.parametrize("dtype,D,Hq,Hkv", [(torch.float32, 128, 12, 4), (torch.bfloat16, 128, 68, 4), (torch.float32, 128, 6, 1),
                                             (torch.float16, 64, 9, 3), (torch.float32, 96, 15, 3), (torch.float32, 128, 28, 2),
                                             (torch.bfloat16, 256, 22, 2)])
def test_any_gqa_group_size(sb, dev, dtype, D, Hq, Hkv):
    """Groups of 3, 17, 6, 3, 5, 14 and 11 query heads per kv head: beyond the matrix-core kernels' 16, or not among
    the vector kernel's built sizes (1, 2, 4, 7, 8), a group is served as several workgroups of a built size."""
    bs, wl = 16, 90
    lens = [1, 16, 17, 65, 129, 300]
    kv, tables = paged_problem(lens, bs, Hkv, D, dtype, seed=Hq)
    q = torch.randn(len(lens), Hq, D, generator=torch.Generator().manual_seed(3)).to(dtype)
    slopes = [2.0 ** (-8.0 * (h + 1) / Hq) for h in range(Hq)]
    for n_split, opts in ((1, {}), (3, dict(alibi_slopes=torch.tensor(slopes, device=dev)))):
        out = sb.ops.swa_decode_attention(q.to(dev), kv[0].to(dev), kv[1].to(dev), torch.tensor(lens, dtype=torch.int32, device=dev),
                                          block_table=tables.to(dev), window_left=wl, scale=D ** -0.5, n_split=n_split, **opts)
        ref = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(), lens,
                                       D ** -0.5, wl, alibi_slopes=slopes if opts else None)
        tol = 1e-4 if (dtype == torch.float32 and opts) else TOL[dtype]
        assert np.abs(out.float().cpu().numpy() - ref).max() <= tol, (n_split, bool(opts))


def test_what_stays_at_128(sb, dev):
    with pytest.raises(ValueError, match="Head size"):
        sb.MetaAttentionImpl(8, 100, 1.0, 2, None, 65, "auto")
    with pytest.raises(NotImplementedError, match="head size 128"):
        sb.MetaAttentionImpl(8, 64, 1.0, 2, None, 65, "fp8")
    q = torch.randn(4, 8, 48, device=dev)
    kc = torch.randn(4, 16, 2, 48, device=dev)
    with pytest.raises((ValueError, NotImplementedError, RuntimeError)):
        sb.ops.swa_decode_attention(q, kc, kc, torch.ones(4, dtype=torch.int32, device=dev),
                                    block_table=torch.zeros(4, 1, dtype=torch.int32, device=dev), window_left=8)
