"""Window-bounded paged/dense single-query attention vs the float64 oracle.
Tolerance (BASELINE): max-abs 2e-2 for bf16, 1e-5 for fp32, against fp32/fp64 mathematics."""
import numpy as np
import pytest
import torch

from oracle import attention as A

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3, torch.float32: 1e-5}


def paged_problem(lens, bs, Hkv, D, dtype, seed, slack=5, resident_from=None):
    """Random paged cache holding `lens[b]` keys per sequence in a seeded block permutation."""
    g = torch.Generator().manual_seed(seed)
    need = [(n + bs - 1) // bs for n in lens]
    nb = sum(need) + slack
    perm = torch.randperm(nb, generator=g)
    kv = torch.randn(2, nb, bs, Hkv, D, generator=g).to(dtype)
    tables = torch.zeros(len(lens), max(max(need), 1), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
    return kv, tables


def run_paged(sb, dev, q, kv, tables, lens, wl, scale, **kw):
    return sb.ops.swa_decode_attention(q.to(dev), kv[0].to(dev), kv[1].to(dev),
                                       torch.tensor(lens, dtype=torch.int32, device=dev),
                                       block_table=tables.to(dev), window_left=wl, scale=scale, **kw)


@pytest.mark.parametrize("dtype,force_valu", [(torch.bfloat16, False), (torch.float16, False), (torch.float32, False),
                                              (torch.bfloat16, True)])
@pytest.mark.parametrize("Hq,Hkv", [(28, 4), (8, 8), (8, 2), (16, 2)])
@pytest.mark.parametrize("wl,n_split", [(64, 1), (64, 3), (37, 0), (-1, 2), (0, 1)])
def test_paged_decode_vs_oracle(sb, dev, dtype, force_valu, Hq, Hkv, wl, n_split):
    D, bs = 128, 16
    lens = [1, 15, 16, 17, 64, 65, 100, 129, 200]
    kv, tables = paged_problem(lens, bs, Hkv, D, dtype, seed=Hq * 7 + (wl % 5))
    g = torch.Generator().manual_seed(2)
    q = torch.randn(len(lens), Hq, D, generator=g).to(dtype)
    scale = D ** -0.5
    out, lse = run_paged(sb, dev, q, kv, tables, lens, wl, scale, n_split=n_split, return_lse=True, force_valu=force_valu)
    ref, ref_lse = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(),
                                            tables.numpy(), lens, scale, wl, return_lse=True)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= TOL[dtype]
    assert np.abs(lse.cpu().numpy() - ref_lse).max() <= 1e-3


@pytest.mark.parametrize("Hq,Hkv", [(12, 4), (5, 1), (16, 1), (26, 2)])
def test_matrix_core_kernel_any_group_size(sb, dev, Hq, Hkv):
    D, bs = 128, 16
    lens = [1, 31, 32, 33, 95, 257]
    kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, seed=Hq)
    q = torch.randn(len(lens), Hq, D, generator=torch.Generator().manual_seed(4)).bfloat16()
    for wl, n_split in [(50, 1), (-1, 3), (31, 2)]:
        out = run_paged(sb, dev, q, kv, tables, lens, wl, D ** -0.5, n_split=n_split)
        ref = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(),
                                       tables.numpy(), lens, D ** -0.5, wl)
        assert np.abs(out.float().cpu().numpy() - ref).max() <= 2e-2


def test_uninitialised_rows_outside_the_window_do_not_leak(sb, dev):
    """Rows past the newest key and rows older than the window may hold anything (NaN bit
    patterns included): they must not reach the output."""
    D, bs, Hq, Hkv, wl = 128, 16, 28, 4, 40
    lens = [70, 21]
    kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, seed=9)
    q = torch.randn(2, Hq, D, generator=torch.Generator().manual_seed(5)).bfloat16()
    ref = run_paged(sb, dev, q, kv, tables, lens, wl, D ** -0.5)
    poisoned = kv.clone()
    for b, n in enumerate(lens):
        for i in list(range(0, max(0, n - 1 - wl))) + list(range(n, tables.shape[1] * bs)):
            blk = int(tables[b, i // bs])
            if i // bs < (n + bs - 1) // bs or i < n:
                poisoned[:, blk, i % bs] = float("nan")
    for fv in (False, True):
        out = run_paged(sb, dev, q, poisoned, tables, lens, wl, D ** -0.5, force_valu=fv)
        assert not torch.isnan(out).any()
        assert (out.float() - ref.float()).abs().max() <= 4e-3


def test_block_size_64_and_large_scores(sb, dev):
    # run_model_vllm.py uses block_size 64; scores up to ~|40| exercise the running-max rescale
    D, bs, Hq, Hkv = 128, 64, 28, 4
    lens = [300, 64, 5]
    kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, seed=3)
    q = (torch.randn(3, Hq, D, generator=torch.Generator().manual_seed(1)) * 4).bfloat16()
    out = run_paged(sb, dev, q, kv, tables, lens, 100, 1.0 / 3, n_split=2)
    ref = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(),
                                   tables.numpy(), lens, 1.0 / 3, 100)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= 2e-2


def test_empty_rows_key_lo_and_row_seq(sb, dev):
    """seq_len 0 and key_lo beyond the query give zeros; several query rows may share a sequence
    (varlen decode): row r sees the first seq_lens[r] keys of sequence row_seq[r]."""
    D, bs, Hq, Hkv, wl = 128, 16, 28, 4, 20
    lens = [50, 33]
    kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, seed=5)
    row_seq = [0, 0, 0, 1, 1, 0]
    row_len = [48, 49, 50, 33, 0, 50]
    key_lo = [0, 40, 0, 0, 0, 50]
    g = torch.Generator().manual_seed(3)
    q = torch.randn(len(row_seq), Hq, D, generator=g).bfloat16()
    out, lse = sb.ops.swa_decode_attention(
        q.to(dev), kv[0].to(dev), kv[1].to(dev), torch.tensor(row_len, dtype=torch.int32, device=dev),
        block_table=tables.to(dev), row_seq=torch.tensor(row_seq, dtype=torch.int32, device=dev),
        key_lo=torch.tensor(key_lo, dtype=torch.int32, device=dev), window_left=wl, n_split=2, return_lse=True)
    out = out.float().cpu().numpy()
    k_np, v_np = kv[0].float().numpy(), kv[1].float().numpy()
    for r in range(len(row_seq)):
        n, s = row_len[r], row_seq[r]
        lo = max(max(0, n - 1 - wl), key_lo[r])
        if n == 0 or lo >= n:
            assert (out[r] == 0).all() and torch.isinf(lse[r]).all() and (lse[r] < 0).all()
            continue
        kk = A.gather_paged(k_np, tables[s].numpy(), n); vv = A.gather_paged(v_np, tables[s].numpy(), n)
        masked = (np.arange(n) < lo)[None]
        for h in range(Hq):
            ref = A.masked_softmax_attention(q[r, h].float().numpy()[None], kk[:, h // 7], vv[:, h // 7], masked, D ** -0.5)
            assert np.abs(out[r, h] - ref[0]).max() <= 2e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_mode_matches_paged_semantics(sb, dev, dtype):
    """Dense [B, Hkv, cap, D] storage with a row window (the HF cache layout)."""
    B, Hq, Hkv, D, cap, start, L, W = 3, 28, 4, 128, 96, 11, 70, 32
    g = torch.Generator().manual_seed(6)
    store_k = torch.randn(B, Hkv, cap, D, generator=g).to(dtype).to(dev)
    store_v = torch.randn(B, Hkv, cap, D, generator=g).to(dtype).to(dev)
    k, v = store_k[:, :, start:start + L], store_v[:, :, start:start + L]
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    kv_start = torch.arange(B, dtype=torch.int64, device=dev) * (Hkv * cap)
    out = sb.ops.swa_decode_attention(
        q.to(dev), k, v, torch.full((B,), L, dtype=torch.int32, device=dev), kv_start=kv_start,
        kv_strides=(0, k.stride(2), k.stride(1)), num_kv_heads=Hkv, window_left=W - 1, max_seq_len=L)
    ref = A.sdpa_window_attention(q.float().numpy()[:, :, None], k.float().cpu().numpy(), v.float().cpu().numpy(), W)
    assert np.abs(out.float().cpu().numpy() - ref[:, :, 0]).max() <= TOL[dtype]


def config2_problem(dev, B=64, seed=0):
    """BASELINE config 2: B=64, 28q/4kv, D=128, bs=16, window_left=4096, ctx ~ U[1024, 32768],
    only in-window blocks resident, seeded block permutation, bf16 N(0,1)."""
    Hq, Hkv, D, bs, wl = 28, 4, 128, 16, 4096
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(1024, 32769, (B,), generator=g)
    pos = ctx                                   # position of the new token
    lo_blk = torch.clamp((pos - wl) // bs, min=0)
    hi_blk = pos // bs
    nblk = (hi_blk - lo_blk + 1)
    nb = int(nblk.sum() * 1.1) + 1
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(B, int(nblk.max()), dtype=torch.int32)
    p = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[p:p + nblk[b]]; p += int(nblk[b])
    seqlens = (pos + 1 - lo_blk * bs).to(torch.int32)
    kv = torch.randn(2, nb, bs, Hkv, D, device=dev, dtype=torch.bfloat16)
    q = torch.randn(B, Hq, D, device=dev, dtype=torch.bfloat16)
    return dict(q=q, kv=kv, tables=tables.to(dev), seqlens=seqlens.to(dev), wl=wl, D=D, Hq=Hq, Hkv=Hkv, bs=bs)


def test_config2_full_size_properties(sb, dev):
    """Full BASELINE config 2 through size-independent properties plus a sampled oracle check."""
    p = config2_problem(dev)
    q, kv, tables, seqlens, wl = p["q"], p["kv"], p["tables"], p["seqlens"], p["wl"]
    base = sb.ops.swa_decode_attention(q, kv[0], kv[1], seqlens, block_table=tables, window_left=wl)
    # (1) the split count does not change the result beyond fp32 merge rounding
    one = sb.ops.swa_decode_attention(q, kv[0], kv[1], seqlens, block_table=tables, window_left=wl, n_split=1)
    many = sb.ops.swa_decode_attention(q, kv[0], kv[1], seqlens, block_table=tables, window_left=wl, n_split=16)
    assert (base.float() - one.float()).abs().max() <= 4e-3 and (base.float() - many.float()).abs().max() <= 4e-3
    # (2) relabelling physical blocks leaves the result bit-identical
    nb = kv.shape[1]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1)).to(dev)
    inv = torch.argsort(perm)
    moved = sb.ops.swa_decode_attention(q, kv[0][perm], kv[1][perm], seqlens, block_table=inv[tables.long()].int(),
                                        window_left=wl)
    assert torch.equal(moved, base)
    # (3) constant V gives that constant
    const_v = torch.full_like(kv[1], 0.75)
    out = sb.ops.swa_decode_attention(q, kv[0], const_v, seqlens, block_table=tables, window_left=wl)
    assert (out.float() - 0.75).abs().max() <= 4e-3
    # (4) a few sequences against the oracle (shortest, longest, first), on their own blocks only
    sl = seqlens.cpu()
    for b in sorted({0, int(sl.argmin()), int(sl.argmax())}):
        n = int(sl[b])
        nblk = (n + p["bs"] - 1) // p["bs"]
        blocks = tables[b, :nblk].long()
        kk, vv = kv[0][blocks].float().cpu().numpy(), kv[1][blocks].float().cpu().numpy()
        ref = A.paged_decode_attention(q[b:b + 1].float().cpu().numpy(), kk, vv, np.arange(nblk)[None], [n],
                                       p["D"] ** -0.5, wl)
        assert np.abs(base[b:b + 1].float().cpu().numpy() - ref).max() <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("wl,n_split", [(40, 1), (40, 3), (-1, 2), (0, 1)])
def test_fused_append_equals_append_then_attend(sb, dev, dtype, wl, n_split):
    """One launch that appends the newest K/V row and attends == kv_append followed by attention:
    identical cache bytes and identical output bits; padded rows (slot -1) store nothing.
    (fp32 takes the vector-ALU kernel, where the same call runs the two launches internally.)"""
    D, bs, Hq, Hkv = 128, 16, 28, 4
    lens = [1, 16, 17, 33, 64, 100, 129]                      # includes a new token that opens a block
    kv, tables = paged_problem(lens, bs, Hkv, D, dtype, seed=11)
    g = torch.Generator().manual_seed(8)
    R = len(lens)
    q = torch.randn(R, Hq, D, generator=g).to(dtype).to(dev)
    k_new = torch.randn(R, Hkv, D, generator=g).to(dtype).to(dev)
    v_new = torch.randn(R, Hkv, D, generator=g).to(dtype).to(dev)
    pos = torch.tensor(lens) - 1
    slots = (tables[torch.arange(R), (pos // bs)].long() * bs + pos % bs)
    slots[3] = -1                                              # a padded lane
    slots = slots.to(dev)
    sl = torch.tensor(lens, dtype=torch.int32, device=dev)
    a = kv.clone().to(dev)
    sb.ops.kv_append(k_new, v_new, a[0], a[1], slots)
    ref = sb.ops.swa_decode_attention(q, a[0], a[1], sl, block_table=tables.to(dev), window_left=wl, n_split=n_split)
    b = kv.clone().to(dev)
    out = sb.ops.swa_decode_attention(q, b[0], b[1], sl, block_table=tables.to(dev), window_left=wl, n_split=n_split,
                                      new_key=k_new, new_value=v_new, new_slot_mapping=slots)
    live = [r for r in range(R) if r != 3]                     # the output of a padded lane is unspecified
    assert torch.equal(out[live], ref[live])
    assert torch.equal(a, b)                                   # same cache bytes, padded lane stored nothing
    with pytest.raises(ValueError, match="go together"):
        sb.ops.swa_decode_attention(q, b[0], b[1], sl, block_table=tables.to(dev), new_key=k_new)
    with pytest.raises(ValueError, match="paged mode"):
        sb.ops.swa_decode_attention(q, b[0], b[1], sl, block_table=tables.to(dev), row_seq=sl, new_key=k_new,
                                    new_value=v_new, new_slot_mapping=slots)


def test_argument_errors(sb, dev):
    q = torch.zeros(2, 28, 128, device=dev, dtype=torch.bfloat16)
    kv = torch.zeros(2, 4, 16, 4, 128, device=dev, dtype=torch.bfloat16)
    sl = torch.ones(2, dtype=torch.int32, device=dev)
    bt = torch.zeros(2, 1, dtype=torch.int32, device=dev)
    with pytest.raises(ValueError, match="int32"):
        sb.ops.swa_decode_attention(q, kv[0], kv[1], sl.long(), block_table=bt)
    with pytest.raises(ValueError, match="share one dtype"):
        sb.ops.swa_decode_attention(q.float(), kv[0], kv[1], sl, block_table=bt)
    with pytest.raises(ValueError, match="multiple"):                 # 27 query heads over 4 kv heads
        sb.ops.swa_decode_attention(torch.zeros(2, 27, 128, device=dev, dtype=torch.bfloat16), kv[0], kv[1], sl, block_table=bt)
    with pytest.raises(ValueError, match="dense mode"):
        sb.ops.swa_decode_attention(q, kv[0], kv[1], sl)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", ["ragged", "many_rows", "tiny", "one_row"])
def test_balanced_split_vs_oracle_and_fixed_split(sb, dev, dtype, case):
    """The balanced split (runs of chunks cut across row boundaries) against the oracle and
    against the fixed split, with rows that take a fraction of a run, rows that take several,
    empty rows, more than 64 rows (two passes of the row scan), and a fused append."""
    Hq, Hkv, D, bs = 28, 4, 128, 16
    g = torch.Generator().manual_seed({"ragged": 1, "many_rows": 2, "tiny": 3, "one_row": 4}[case])
    if case == "ragged":
        lens, wl, n_split = [1, 700, 33, 0, 2049, 5, 64, 1300, 31, 32, 900, 0], 1023, 4
    elif case == "many_rows":
        lens, wl, n_split = [int(x) for x in torch.randint(0, 400, (150,), generator=g)], 255, 3
    elif case == "tiny":
        lens, wl, n_split = [3, 1, 2], -1, 5          # fewer chunks than workgroups
    else:
        lens, wl, n_split = [4000], 2047, 16
    B = len(lens)
    kv, tables = paged_problem(lens, bs, Hkv, D, dtype, 11)
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    scale = D ** -0.5
    ref, ref_lse = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(),
                                            tables.numpy(), lens, scale, wl, return_lse=True)
    out, lse = run_paged(sb, dev, q, kv, tables, lens, wl, scale, n_split=n_split, balanced=True, return_lse=True)
    fixed = run_paged(sb, dev, q, kv, tables, lens, wl, scale, n_split=n_split, balanced=False)
    got = out.float().cpu().numpy()
    live = [b for b in range(B) if lens[b] > 0]
    dead = [b for b in range(B) if lens[b] == 0]
    assert np.abs(got[live] - ref[live]).max() <= TOL[dtype]
    assert np.abs(lse.cpu().numpy()[live] - ref_lse[live]).max() <= 2e-3
    assert (got[dead] == 0).all() and np.isneginf(lse.cpu().numpy()[dead]).all()
    assert (out.float() - fixed.float()).abs().max().item() <= 4e-3
    # the same call twice gives the same bits (no dependence on workgroup arrival order)
    again = run_paged(sb, dev, q, kv, tables, lens, wl, scale, n_split=n_split, balanced=True)
    assert torch.equal(again, out)


def test_balanced_split_fused_append(sb, dev):
    """Fused append under the balanced split: cache and output equal append-then-attend."""
    Hq, Hkv, D, bs, wl = 28, 4, 128, 16, 300
    lens = [17, 301, 1200, 1, 640, 333, 96, 2000]
    B = len(lens)
    g = torch.Generator().manual_seed(5)
    kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, 13)
    q = torch.randn(B, Hq, D, generator=g).bfloat16().to(dev)
    nk, nv = (torch.randn(B, Hkv, D, generator=g).bfloat16().to(dev) for _ in range(2))
    slots = torch.tensor([int(tables[b, (lens[b] - 1) // bs]) * bs + (lens[b] - 1) % bs for b in range(B)],
                         dtype=torch.int64, device=dev)
    slots[3] = -1                                       # padded row: nothing stored
    sl = torch.tensor(lens, dtype=torch.int32, device=dev)
    a, b_ = kv.clone().to(dev), kv.clone().to(dev)
    sb.ops.kv_append(nk, nv, a[0], a[1], slots)
    ref = sb.ops.swa_decode_attention(q, a[0], a[1], sl, block_table=tables.to(dev), window_left=wl, n_split=4, balanced=False)
    out = sb.ops.swa_decode_attention(q, b_[0], b_[1], sl, block_table=tables.to(dev), window_left=wl, n_split=4,
                                      balanced=True, new_key=nk, new_value=nv, new_slot_mapping=slots)
    assert torch.equal(a, b_)
    keep = [b for b in range(B) if b != 3]              # row 3's newest key is in neither cache
    assert (out[keep].float() - ref[keep].float()).abs().max().item() <= 4e-3


def test_split_policy_from_host_lengths(sb, dev):
    """With host_seq_lens the op decides fixed/balanced itself: a ragged batch takes the balanced
    split (bit-identical to asking for it), an even one the fixed split."""
    Hq, Hkv, D, bs = 28, 4, 128, 16
    g = torch.Generator().manual_seed(8)
    for lens, expect in (([6000] + [200] * 15, True), ([1500] * 16, False)):
        kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, 17)
        q = torch.randn(len(lens), Hq, D, generator=g).bfloat16()
        n_split = sb._native.lib().sb_swa_decode_auto_split(len(lens), Hkv, max(lens), -1)
        assert n_split > 1
        assert sb.ops.plan_decode_split(len(lens), Hkv, max(lens), -1, lens) is expect
        auto = run_paged(sb, dev, q, kv, tables, lens, -1, D ** -0.5, max_seq_len=max(lens), host_seq_lens=lens)
        forced = run_paged(sb, dev, q, kv, tables, lens, -1, D ** -0.5, max_seq_len=max(lens), balanced=expect)
        assert torch.equal(auto, forced)


@pytest.mark.parametrize("n_split", [1, 3, 7])
@pytest.mark.parametrize("wl", [-1, 100, 1000])
def test_prefetch_depths_and_segment_ends_agree(sb, dev, wl, n_split):
    """The streaming loop exists in three prefetch depths (flag bits 4-6); a segment's head chunk is fetched
    first and its tail chunk two chunks before the stream ends, whatever the depth and however few interior
    chunks the segment has (lengths here give segments of 0, 1, 2, 3 and many interior chunks). Every depth
    must give the depth-1 result bit for bit (same arithmetic in the same order), and that one the oracle's."""
    Hq, Hkv, D, bs = 28, 4, 128, 16
    lens = [1, 31, 32, 33, 64, 65, 97, 129, 161, 200, 449, 1500, 2047]
    kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, 23)
    g = torch.Generator().manual_seed(wl + n_split)
    q = torch.randn(len(lens), Hq, D, generator=g).bfloat16()
    outs = [run_paged(sb, dev, q, kv, tables, lens, wl, D ** -0.5, n_split=n_split, balanced=False,
                      pipeline_depth=depth) for depth in (1, 2, 3)]
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    ref = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(),
                                   lens, D ** -0.5, wl)
    assert np.abs(outs[0].float().cpu().numpy() - ref).max() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,n_split,wl", [(1, 2, -1), (7, 3, 300), (8, 4, 300), (21, 5, 97), (64, 4, 4096), (130, 2, -1)])
def test_merge_inside_the_split_kernel_equals_merge_kernel(sb, dev, dtype, rows, n_split, wl):
    """With merge_in_kernel the matrix-core fixed split merges its partial results itself (the last wavefront of a
    row to finish does it); without, the same partials go through the merge kernel. Same arithmetic in the same
    order: outputs and log-sum-exps must agree bit for bit, for row counts that are and are not multiples of 8
    (the launch pads them), with empty rows, and the arrival counters must be back at zero afterwards."""
    D, bs, Hq, Hkv = 128, 16, 28, 4
    g = torch.Generator().manual_seed(rows * 31 + n_split)
    lens = torch.randint(1, 900, (rows,), generator=g).tolist()
    if rows > 2:
        lens[1] = 0                                             # a row with nothing to attend to
    kv, tables = paged_problem([max(n, 1) for n in lens], bs, Hkv, D, dtype, seed=rows)
    q = torch.randn(rows, Hq, D, generator=g).to(dtype)
    outs = []
    for inside in (True, False):
        outs.append(run_paged(sb, dev, q, kv, tables, lens, wl, D ** -0.5, n_split=n_split, return_lse=True,
                              merge_in_kernel=inside, balanced=False))
    assert torch.equal(outs[0][0].view(torch.int16), outs[1][0].view(torch.int16))
    assert torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32))
    ref = A.paged_decode_attention(q.float().numpy(), kv[0].float().numpy(), kv[1].float().numpy(), tables.numpy(), lens,
                                   D ** -0.5, wl)
    assert np.abs(outs[0][0].float().cpu().numpy() - ref).max() <= TOL[dtype]
    ws = sb.ops._workspace(dev, 1 << 16)                        # this stream's scratch: its first 64 KiB are the counters
    torch.cuda.synchronize()
    assert not ws[:1 << 16].any(), "arrival counters (or the XCD fault word) left non-zero"


def test_merge_inside_the_split_kernel_many_launches_back_to_back(sb, dev):
    """Counters re-arm themselves: many launches in a row on one workspace, alternating shapes, no host
    synchronisation in between, each checked against its merge-kernel twin afterwards."""
    D, bs, Hq, Hkv = 128, 16, 28, 4
    probs = []
    for i, (rows, n_split) in enumerate([(64, 4), (9, 7), (33, 2), (64, 8)]):
        g = torch.Generator().manual_seed(100 + i)
        lens = torch.randint(200, 1500, (rows,), generator=g).tolist()
        kv, tables = paged_problem(lens, bs, Hkv, D, torch.bfloat16, seed=i)
        q = torch.randn(rows, Hq, D, generator=g).bfloat16()
        probs.append((q.to(dev), kv.to(dev), tables.to(dev), torch.tensor(lens, dtype=torch.int32, device=dev), n_split))
    call = lambda pr, inside: sb.ops.swa_decode_attention(pr[0], pr[1][0], pr[1][1], pr[3], block_table=pr[2], window_left=700,
                                                        n_split=pr[4], merge_in_kernel=inside, balanced=False)
    want = [call(pr, False) for pr in probs]
    got = [call(probs[i % 4], True) for i in range(40)]
    torch.cuda.synchronize()
    for i, o in enumerate(got):
        assert torch.equal(o, want[i % 4]), f"launch {i}"


@pytest.mark.parametrize("seed", range(40))
def test_random_shapes_vs_oracle(sb, dev, seed):
    """Seeded random cases across what the decode kernels specialise on: GQA group (1..16 on the matrix cores),
    dtype, block size, window, split count and kind (fixed / balanced / merged inside the kernel), prefetch
    depth, ragged lengths around the 16/32-key boundaries (empty rows included), key_lo, several query rows per
    sequence, the fused append, meta rows, soft cap / ALiBi. Stale cache rows hold NaN."""
    r = np.random.default_rng(2000 + seed)
    D = 128
    Hkv = int(r.choice([1, 2, 4]))
    G = int(r.integers(1, 17))
    Hq = Hkv * G
    dtype = torch.bfloat16 if r.random() < 0.7 else torch.float16
    bs = int(r.choice([16, 32, 48, 64, 128]))
    wl = int(r.choice([-1, 0, 7, 31, 32, 100, 257, 1000]))
    B = int(r.integers(1, 9))
    lens = [int(r.choice([0, 1, 15, 16, 17, 31, 32, 33, 64, 100, 129, 300, 700])) for _ in range(B)]
    n_split = int(r.choice([0, 1, 2, 3, 5]))
    mode = r.choice(["fixed", "balanced", "merge_in_kernel", "fused", "meta", "options", "rows"])
    g = torch.Generator().manual_seed(seed)
    need = [(n + bs - 1) // bs for n in lens]
    nb = sum(need) + 2
    perm = torch.randperm(nb, generator=g)
    kc = torch.full((nb, bs, Hkv, D), float("nan")).to(dtype); vc = torch.full((nb, bs, Hkv, D), float("nan")).to(dtype)
    tables = torch.zeros(B, max(max(need), 1), dtype=torch.int32)
    ks, vs = [], []
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
        k = torch.randn(lens[b], Hkv, D, generator=g).to(dtype); v = torch.randn(lens[b], Hkv, D, generator=g).to(dtype)
        ks.append(k); vs.append(v)
        for i in range(lens[b]):
            kc[int(tables[b, i // bs]), i % bs] = k[i]; vc[int(tables[b, i // bs]), i % bs] = v[i]
    scale = D ** -0.5
    kw = dict(n_split=n_split, pipeline_depth=int(r.choice([0, 1, 2, 3])))
    rows = list(range(B))                      # sequence of each query row
    row_len = list(lens)                       # keys visible to each row
    key_lo = None
    slopes, softcap, meta = None, 0.0, None
    if mode == "balanced":
        kw["balanced"] = True
    elif mode == "merge_in_kernel":
        kw.update(balanced=False, merge_in_kernel=True)
    elif mode == "options":
        slopes = [float(2.0 ** (-8.0 * (h + 1) / Hq)) for h in range(Hq)]
        softcap = float(r.choice([0.0, 2.0]))
        kw.update(softcap=softcap, alibi_slopes=torch.tensor(slopes, device=dev))
    elif mode == "meta":
        M = int(r.choice([1, 32, 100]))
        meta = (torch.randn(M, Hkv, D, generator=g).to(dtype), torch.randn(M, Hkv, D, generator=g).to(dtype))
        kw.update(meta_k=meta[0].to(dev), meta_v=meta[1].to(dev), balanced=False)
    elif mode == "rows":                       # several rows per sequence, each with its own length and key_lo
        rows = [int(r.integers(0, B)) for _ in range(B + 3)]
        row_len = [int(r.integers(0, lens[s] + 1)) for s in rows]
        key_lo = [int(r.integers(0, 40)) if r.random() < 0.5 else 0 for _ in rows]
        kw.update(row_seq=torch.tensor(rows, dtype=torch.int32, device=dev),
                  key_lo=torch.tensor(key_lo, dtype=torch.int32, device=dev), max_seq_len=max(lens + [1]))
    R = len(rows)
    q = torch.randn(R, Hq, D, generator=g).to(dtype)
    kc_d, vc_d = kc.to(dev), vc.to(dev)
    if mode == "fused":                        # the newest key of every non-empty row arrives with the call
        newk = torch.zeros(B, Hkv, D, dtype=dtype); newv = torch.zeros(B, Hkv, D, dtype=dtype)
        slots = torch.full((B,), -1, dtype=torch.int64)
        for b, n in enumerate(lens):
            if n > 0:
                newk[b], newv[b] = ks[b][n - 1], vs[b][n - 1]
                blk, off = int(tables[b, (n - 1) // bs]), (n - 1) % bs
                slots[b] = blk * bs + off
                kc_d[blk, off] = float("nan"); vc_d[blk, off] = float("nan")
        kw.update(new_key=newk.to(dev), new_value=newv.to(dev), new_slot_mapping=slots.to(dev))
        if min(lens) == 0:                     # (a row without keys has no newest key to append)
            pytest.skip("fused append needs a key in every row")
    out = sb.ops.swa_decode_attention(q.to(dev), kc_d, vc_d, torch.tensor(row_len, dtype=torch.int32, device=dev),
                                      block_table=tables.to(dev), window_left=wl, scale=scale, **kw).float().cpu().numpy()
    assert np.isfinite(out).all()
    for i, s in enumerate(rows):
        n = row_len[i]
        lo = max(0 if wl < 0 else max(0, n - 1 - wl), key_lo[i] if key_lo else 0)
        kk, vv = ks[s][lo:n].float().numpy(), vs[s][lo:n].float().numpy()
        for h in range(Hq):
            kh, vh = kk[:, h // G], vv[:, h // G]
            bias = None
            if slopes is not None:
                bias = -slopes[h] * (n - 1 - np.arange(lo, n))[None]
            if meta is not None:
                kh = np.concatenate([meta[0].float().numpy()[:, h // G], kh]); vh = np.concatenate([meta[1].float().numpy()[:, h // G], vh])
            if len(kh) == 0:
                assert (out[i, h] == 0).all()
                continue
            ref = A.masked_softmax_attention(q[i, h].float().numpy()[None], kh, vh, np.zeros((1, len(kh)), bool), scale,
                                             softcap=softcap, bias=bias)[0]
            err = np.abs(out[i, h] - ref).max()
            assert err <= TOL[dtype], (err, dict(seed=seed, mode=str(mode), Hq=Hq, Hkv=Hkv, bs=bs, wl=wl, lens=lens, n_split=n_split))
    if mode == "fused":                        # and the cache now holds them
        for b, n in enumerate(lens):
            blk, off = int(tables[b, (n - 1) // bs]), (n - 1) % bs
            assert torch.equal(kc_d[blk, off].cpu(), ks[b][n - 1]) and torch.equal(vc_d[blk, off].cpu(), vs[b][n - 1])
