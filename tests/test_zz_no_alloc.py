"""sb_swa_decode_static (split-K partials in the library's own device array, no allocation) against
sb_swa_decode with a caller workspace: both called straight through the C ABI, outputs and
log-sum-exps bit-identical (same kernels, same summation order). Two calls in a row share the
array, the second with a smaller input, so stale partials of the first are in it."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _problem(lens, bs, Hkv, D, seed):
    g = torch.Generator().manual_seed(seed)
    need = [(n + bs - 1) // bs for n in lens]
    nb = sum(need) + 3
    perm = torch.randperm(nb, generator=g)
    kv = torch.randn(2, nb, bs, Hkv, D, generator=g).bfloat16()
    tables = torch.zeros(len(lens), max(need), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]
        p += n
    return kv, tables


def _args(N, q, kv, tables, seq_lens, out, lse, wl, n_split, flags, ws):
    Hq, D = q.shape[1], q.shape[2]
    kc, vc = kv[0], kv[1]
    return N.SwaDecodeArgs(
        q=N.ptr(q), k_cache=N.ptr(kc), v_cache=N.ptr(vc), out=N.ptr(out), lse=N.ptr(lse),
        block_table=N.ptr(tables), seq_lens=N.ptr(seq_lens),
        workspace=N.ptr(ws), workspace_bytes=0 if ws is None else ws.numel(),
        num_rows=q.shape[0], num_q_heads=Hq, num_kv_heads=kc.shape[2], head_size=D, block_size=kc.shape[1],
        window_left=wl, max_seq_len=tables.shape[1] * kc.shape[1], n_split=n_split, dtype=N.SB_BF16, phases=0,
        flags=flags, scale=D ** -0.5,
        q_stride_row=q.stride(0), q_stride_head=q.stride(1),
        out_stride_row=out.stride(0), out_stride_head=out.stride(1),
        kv_stride_block=kc.stride(0), kv_stride_row=kc.stride(1), kv_stride_head=kc.stride(2),
        block_table_stride=tables.stride(0), stream=N.stream_ptr(q.device))


@pytest.mark.parametrize("flags", [0, 2])  # fixed split, balanced split (SB_DECODE_BALANCED)
def test_static_scratch_matches_workspace_call_twice(sb, dev, flags):
    N = sb._native
    L = N.lib()
    Hq, Hkv, D, bs, wl = 28, 4, 128, 16, 300
    for lens, n_split, seed in (([700, 333, 64, 1, 512, 290, 451, 97, 640, 18, 200, 305], 4, 1),
                                ([90, 411, 33], 3, 2)):        # second call: fewer rows, fewer splits
        kv, tables = _problem(lens, bs, Hkv, D, seed)
        q = torch.randn(len(lens), Hq, D, generator=torch.Generator().manual_seed(seed + 10)).bfloat16().to(dev)
        kv, tables = kv.to(dev), tables.to(dev)
        seq_lens = torch.tensor(lens, dtype=torch.int32, device=dev)
        need = L.sb_swa_decode_workspace_bytes(len(lens), Hq, D, n_split)
        assert 0 < need <= N.SB_SWA_DECODE_STATIC_SCRATCH_BYTES
        ws = torch.zeros(need, dtype=torch.uint8, device=dev)      # a workspace starts zeroed (merge counters)
        outs = []
        for fn, w in ((L.sb_swa_decode, ws), (L.sb_swa_decode_static, None)):
            out = torch.full((len(lens), Hq, D), float("nan"), dtype=torch.bfloat16, device=dev)
            lse = torch.full((len(lens), Hq), float("nan"), dtype=torch.float32, device=dev)
            a = _args(N, q, kv, tables, seq_lens, out, lse, wl, n_split, flags, w)
            rc = fn(C.byref(a))
            assert rc == 0, N.last_error()
            torch.cuda.synchronize()
            outs.append((out, lse))
        assert torch.equal(outs[0][0].view(torch.int16), outs[1][0].view(torch.int16))
        assert torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32))
        assert not torch.isnan(outs[1][0].float()).any()


def test_static_scratch_rejects_oversized_call(sb, dev):
    N = sb._native
    L = N.lib()
    rows, Hq, Hkv, D, n_split = 600, 28, 4, 128, 8
    assert L.sb_swa_decode_workspace_bytes(rows, Hq, D, n_split) > N.SB_SWA_DECODE_STATIC_SCRATCH_BYTES
    kv, tables = _problem([40] * rows, 16, Hkv, D, 3)
    q = torch.zeros(rows, Hq, D, dtype=torch.bfloat16, device=dev)
    out = torch.zeros_like(q)
    a = _args(N, q, kv.to(dev), tables.to(dev), torch.full((rows,), 40, dtype=torch.int32, device=dev), out, None,
              -1, n_split, 0, None)
    assert L.sb_swa_decode_static(C.byref(a)) == N.SB_ERR_WORKSPACE
    assert "scratch" in N.last_error()
