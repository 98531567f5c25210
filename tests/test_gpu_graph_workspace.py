"""The split-K scratch of a captured decode call belongs to the graph: a later, larger eager call must not
replace or free it (the allocator could then hand the block to another tensor while every replay still
writes and merges partials there), and calls on different streams must not share one buffer."""
import numpy as np
import pytest
import torch

from oracle import attention as A

pytestmark = pytest.mark.gpu

HQ, HKV, D, BS = 28, 4, 128, 16


def _problem(dev, lens, seed):
    g = torch.Generator().manual_seed(seed)
    need = [(n + BS - 1) // BS for n in lens]
    nb = sum(need) + 3
    perm = torch.randperm(nb, generator=g)
    kv = torch.randn(2, nb, BS, HKV, D, generator=g).bfloat16()
    tables = torch.zeros(len(lens), max(need), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]
        p += n
    q = torch.randn(len(lens), HQ, D, generator=g).bfloat16()
    return q.to(dev), kv.to(dev), tables.to(dev), torch.tensor(lens, dtype=torch.int32, device=dev)


def test_graph_replays_keep_their_workspace(sb, dev):
    lens = [700, 333, 512, 90, 640, 451]
    q, kv, tables, sl = _problem(dev, lens, 1)
    out = torch.zeros_like(q)
    call = lambda: sb.ops.swa_decode_attention(q, kv[0], kv[1], sl, block_table=tables, window_left=300, n_split=4, out=out)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        call()                                        # warm-up outside the capture, as capture_step does
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    eager = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    ref = A.paged_decode_attention(q.float().cpu().numpy(), kv[0].float().cpu().numpy(), kv[1].float().cpu().numpy(),
                                   tables.cpu().numpy(), lens, D ** -0.5, 300)
    # a larger request on the eager path (more rows, more splits): must leave the graph's buffer alone
    q2, kv2, t2, sl2 = _problem(dev, [900] * 40, 2)
    big = sb.ops.swa_decode_attention(q2, kv2[0], kv2[1], sl2, block_table=t2, window_left=-1, n_split=16)
    torch.cuda.synchronize()
    # fresh tensors of the sizes the allocator would carve out of a released scratch buffer, with known contents
    fill = [torch.full((n,), 7, dtype=torch.uint8, device=dev) for n in (1 << 20, 1 << 20, 3 << 20, 1 << 19, 1 << 21)]
    for rep in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep}"
        assert np.abs(out.float().cpu().numpy() - ref).max() <= 2e-2
        for t in fill:
            assert bool((t == 7).all()), "a replay wrote into memory the graph no longer owned"
        # eager work between the replays, through the same entry point
        again = sb.ops.swa_decode_attention(q2, kv2[0], kv2[1], sl2, block_table=t2, window_left=-1, n_split=16)
        assert torch.equal(again, big)
    # the graph is dropped: its workspace goes back to the allocator through the release hook, once
    ids = sb.ops.graph_workspace_ids(dev)
    assert ids, "the capture should own a workspace"
    del graph
    assert sb.ops.release_graph_workspace(ids[-1], dev) >= 1 << 20
    assert ids[-1] not in sb.ops.graph_workspace_ids(dev)
    assert sb.ops.release_graph_workspace(ids[-1], dev) == 0


def test_streams_do_not_share_a_workspace(sb, dev):
    ops = sb.ops
    s1, s2 = torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)
    with torch.cuda.stream(s1):
        a = ops._workspace(dev, 4096)
        a_again = ops._workspace(dev, 2048)
    with torch.cuda.stream(s2):
        b = ops._workspace(dev, 4096)
    assert a.data_ptr() == a_again.data_ptr() and a.data_ptr() != b.data_ptr()
    assert ops._workspace(dev, 0) is None
