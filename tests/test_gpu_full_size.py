"""BASELINE configs 4 and 5 at their FULL sizes, checked (not only timed): size-independent properties over
every output plus oracle comparisons on sampled pieces, so that indexing that only goes wrong at size (the
8192-workgroup tile numbering of the prompt kernel, 129-chunk windows, the 4 + 3 head split, 256-row
step advance under graph replay over 14 + 14 layers) cannot pass unseen.

Config 4: 16 prompts x 8192 new tokens, window_left 4096, block_size 16, bf16, through
          `MetaAttentionImpl.forward` as a plain prompt run (keys in flight) and as a chunked-prefill run
          (every token stored, keys read back through the block table).
Config 5: B = 256, 28 layers (14 GLA + 14 SWA sharing one block table), window-saturated sequences,
          host-stepped and then >= 33 graph-replayed steps (every sequence recycles a block at least twice)."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle import gla as G
from oracle import paged as P

pytestmark = pytest.mark.gpu

HQ, HKV, D, BS, WL = 28, 4, 128, 16, 4096


# ------------------------------------------------------------------------------------------ config 4
def _config4_inputs(dev, S, L):
    g = torch.Generator(device=dev).manual_seed(0)
    T = S * L
    q = torch.randn(T, HQ, D, device=dev, dtype=torch.bfloat16, generator=g)
    k = torch.randn(T, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    v = torch.randn(T, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    return q, k, v


def _oracle_tile(q, k, v, s, q0, L, n=64):
    """Oracle output for queries q0 .. q0+n-1 of sequence s over the keys they can see (their own slice of the
    in-flight tensors: positions max(0, q0 - WL) .. q0+n-1)."""
    base = s * L
    k0 = max(0, q0 - WL)
    qs = q[base + q0:base + q0 + n].float().cpu().numpy()
    ks = k[base + k0:base + q0 + n].float().cpu().numpy()
    vs = v[base + k0:base + q0 + n].float().cpu().numpy()
    return A.varlen_window_attention(qs, ks, vs, [0, n], [0, ks.shape[0]], D ** -0.5, WL)


@pytest.mark.parametrize("chunked", [False, True], ids=["prompt_inflight_kv", "chunked_paged_kv"])
def test_config4_full_size(sb, dev, chunked):
    S, L = 16, 8192
    T = S * L
    q, k, v = _config4_inputs(dev, S, L)
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, WL + 1, "auto")
    nb = S * ((L if chunked else WL) // BS + 3) + 8
    runner = sb.SwaCacheRunner(1, nb, BS, WL, HKV, D, torch.bfloat16, dev, max_seqs=S, max_chunk_tokens=L)
    model = P.WindowCacheModel(nb, BS, WL)
    for s in range(S):
        runner.add_seq(s)
        model.add_seq(s)
    meta = runner.build_step([(s, L) for s in range(S)], [], chunked_prefill=chunked)
    # (1) slots bit-exact against the brute-force model, for all 131 072 tokens
    slots = []
    for s in range(S):
        slots += model.append_tokens(s, L, True, store_all=chunked)
    slots_t = torch.tensor(slots, dtype=torch.int64)
    assert torch.equal(meta.slot_mapping.cpu(), slots_t)
    stored = slots_t >= 0
    assert int(stored.sum()) == (T if chunked else S * WL)          # plain: only the last window_left tokens get slots
    out = torch.full((T, HQ, D), float("nan"), dtype=torch.bfloat16, device=dev)
    kv_cache = runner.kv_caches[0]
    impl.forward(None, q, k, v, None, None, None, kv_cache, meta, output=out)
    torch.cuda.synchronize()
    assert not torch.isnan(out.float()).any()
    # (2) every byte of the cache: stored rows hold their token's K/V, everything else is untouched (zero)
    exp = torch.zeros_like(kv_cache)
    idx = slots_t[stored].to(dev)
    exp[0].view(-1, HKV, D)[idx] = k[stored.to(dev)]
    exp[1].view(-1, HKV, D)[idx] = v[stored.to(dev)]
    assert torch.equal(kv_cache, exp)
    # ... and a sample of rows against the numpy append (first / window-edge / last tokens of three sequences)
    ok, ov = (np.zeros((nb, BS, HKV, D), np.float32) for _ in range(2))
    sample = [s * L + t for s in (0, 7, 15) for t in (0, 1, L - WL - 1, L - WL, L - WL + 1, L - 2, L - 1)]
    P.kv_append(k[sample].float().cpu().numpy(), v[sample].float().cpu().numpy(), ok, ov, [slots[t] for t in sample])
    for t in sample:
        if slots[t] >= 0:
            b, r = divmod(slots[t], BS)
            assert np.array_equal(kv_cache[0, b, r].float().cpu().numpy(), ok[b, r])
            assert np.array_equal(kv_cache[1, b, r].float().cpu().numpy(), ov[b, r])
    # (3) sampled 64-token tiles against the oracle: first tile, tiles around the window edge (4096), last tile
    for s in (0, 9, 15):
        for q0 in (0, 64, WL - 64, WL - 32, WL, WL + 64, L // 2 + 32, L - 64):
            ref = _oracle_tile(q, k, v, s, q0, L)
            got = out[s * L + q0:s * L + q0 + 64].float().cpu().numpy()
            assert np.abs(got - ref).max() <= 2e-2, f"sequence {s}, tile at {q0}"
    # (4) constant V gives that constant at every one of the 131 072 x 28 outputs (every tile, every head split)
    vc = torch.full_like(v, 0.75)
    runner2 = sb.SwaCacheRunner(1, nb, BS, WL, HKV, D, torch.bfloat16, dev, max_seqs=S, max_chunk_tokens=L)
    for s in range(S):
        runner2.add_seq(s)
    meta2 = runner2.build_step([(s, L) for s in range(S)], [], chunked_prefill=chunked)
    out_c = torch.full_like(out, float("nan"))
    impl.forward(None, q, k, vc, None, None, None, runner2.kv_caches[0], meta2, output=out_c)
    assert (out_c.float() - 0.75).abs().max() <= 4e-3
    if chunked:
        # (5) relabelling the physical blocks leaves every output bit unchanged
        pm = meta.prefill_metadata
        perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1)).to(dev)
        inv = torch.argsort(perm)
        moved = sb.ops.swa_prefill_attention(q, kv_cache[0][perm], kv_cache[1][perm], query_lens=[L] * S, seq_lens_k=[L] * S,
                                             block_table=inv[pm.block_tables.long()].int(), window_left=WL, scale=D ** -0.5)
        assert torch.equal(moved, out)
    else:
        # (5) the same attention with the keys read back from a paged cache instead of the in-flight tensors
        r3 = sb.SwaCacheRunner(1, S * (L // BS + 3) + 8, BS, WL, HKV, D, torch.bfloat16, dev, max_seqs=S, max_chunk_tokens=L)
        for s in range(S):
            r3.add_seq(s)
        m3 = r3.build_step([(s, L) for s in range(S)], [], chunked_prefill=True)
        out3 = torch.empty_like(out)
        impl.forward(None, q, k, v, None, None, None, r3.kv_caches[0], m3, output=out3)
        assert (out3.float() - out.float()).abs().max() <= 4e-3


def test_config4_ragged_lengths_full_size(sb, dev):
    """The ragged variant of config 4: 16 prompts whose lengths sum to 131 072 (from 1 token to 30 000), through
    the same forward; sampled tiles at the start, at the window edge and at the ragged end of each prompt."""
    lens = [1, 63, 64, 65, 4096, 4097, 4160, 8191, 30000, 12345, 9000, 17, 5000, 20000, 16384]
    lens.append(131072 - sum(lens))
    assert lens[-1] > 0 and sum(lens) == 131072
    S, T = len(lens), 131072
    g = torch.Generator(device=dev).manual_seed(3)
    q = torch.randn(T, HQ, D, device=dev, dtype=torch.bfloat16, generator=g)
    k = torch.randn(T, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    v = torch.randn(T, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, WL + 1, "auto")
    nb = sum(min(n, WL) // BS + 3 for n in lens) + 8
    runner = sb.SwaCacheRunner(1, nb, BS, WL, HKV, D, torch.bfloat16, dev, max_seqs=S, max_chunk_tokens=max(lens))
    for s in range(S):
        runner.add_seq(s)
    meta = runner.build_step(list(enumerate(lens)), [])
    out = torch.full((T, HQ, D), float("nan"), dtype=torch.bfloat16, device=dev)
    impl.forward(None, q, k, v, None, None, None, runner.kv_caches[0], meta, output=out)
    assert not torch.isnan(out.float()).any()
    cu = np.cumsum([0] + lens)
    for s, n in enumerate(lens):
        for q0 in sorted({0, max(0, min(n, WL) - 40), max(0, n - 64), max(0, n // 2 - 7)}):
            m = min(64, n - q0)
            k0 = max(0, q0 - WL)
            ref = A.varlen_window_attention(q[cu[s] + q0:cu[s] + q0 + m].float().cpu().numpy(),
                                            k[cu[s] + k0:cu[s] + q0 + m].float().cpu().numpy(),
                                            v[cu[s] + k0:cu[s] + q0 + m].float().cpu().numpy(), [0, m], [0, q0 + m - k0],
                                            D ** -0.5, WL)
            got = out[cu[s] + q0:cu[s] + q0 + m].float().cpu().numpy()
            assert np.abs(got - ref).max() <= 2e-2, f"sequence {s} (length {n}), queries from {q0}"


# ------------------------------------------------------------------------------------------ config 5
def test_config5_full_size_graph_replayed(sb, dev):
    B, LAYERS = 256, 28
    drv = sb.HybridDecodeCache(B, num_layers=LAYERS, device=dev, randomize=True, seed=1)
    # window-saturated sequences at staggered phases of their 16-token blocks (so evictions spread over the steps)
    ctx = [6000 + 37 * s for s in range(B)]
    model = P.WindowCacheModel(drv.num_blocks, BS, WL)
    for s in range(B):
        drv.manager.append_tokens(s, ctx[s], True)
        model.add_seq(s)
        model.append_tokens(s, ctx[s], True)
    n_swa, n_gla = len(drv.swa_layers), len(drv.gla_layers)
    # expected caches, advanced by plain indexed copies with the MODEL's slots; compared in full at the end
    exp_kv = [c.clone() for c in drv.kv_caches]
    sample_b = sorted({0, 101, 255, int(np.argmax([c % BS == 0 for c in ctx[1:]])) + 1})   # incl. one whose next token opens a block
    sample_gla = [0, 6, 13]                      # GLA layer numbers 0, 12, 26
    sample_swa = [0, 7, 13]                      # SWA layer numbers 1, 15, 27
    st_ref = {(j, b): drv.gla_state[j, b].double().cpu().numpy()[None] for j in sample_gla for b in sample_b}
    g = torch.Generator(device=dev).manual_seed(2)
    q = torch.zeros(B, HQ, D, device=dev, dtype=torch.bfloat16)
    k = torch.zeros(B, HKV, D, device=dev, dtype=torch.bfloat16)
    v = torch.zeros(B, HKV, D, device=dev, dtype=torch.bfloat16)
    gq, gk, gv = (torch.zeros(B, HQ, 1, D, device=dev, dtype=torch.bfloat16) for _ in range(3))
    gg = torch.zeros(B, HQ, 1, D, device=dev)
    s_out = [torch.zeros(B, HQ, D, device=dev, dtype=torch.bfloat16) for _ in range(n_swa)]
    g_out = [torch.zeros(B, HQ, 1, D, device=dev, dtype=torch.bfloat16) for _ in range(n_gla)]

    def fresh():
        for t in (q, k, v, gq, gk, gv):
            t.copy_(torch.randn(t.shape, device=dev, dtype=torch.float32, generator=g))
        gg.copy_(torch.nn.functional.logsigmoid(torch.randn(gg.shape, device=dev, generator=g)) / 16)

    def layers(meta):
        for li in range(LAYERS):
            if li % 2 == 0:
                drv.gla_layer(li, gq, gk, gv, gg, out=g_out[li // 2])
            else:
                drv.swa_layer(li, q, k, v, meta, s_out[li // 2])

    def check_step(slot_t, len_t, table_t, tag, deep):
        slots = [model.append_tokens(s, 1, False)[0] for s in range(B)]
        assert slot_t.cpu().tolist() == slots, tag
        views = [model.view(s) for s in range(B)]
        assert len_t.cpu().tolist() == [vw[1] for vw in views], tag
        tab = table_t.cpu().numpy()
        for s, vw in enumerate(views):
            assert tab[s, :len(vw[0])].tolist() == vw[0] and not tab[s, len(vw[0]):].any(), f"{tag}: table row {s}"
        idx = torch.tensor(slots, dtype=torch.int64, device=dev)
        for j in range(n_swa):
            exp_kv[j][0].view(-1, HKV, D)[idx] = k
            exp_kv[j][1].view(-1, HKV, D)[idx] = v
        # GLA oracle for the sampled (layer, sequence) pairs, every step (the recurrence has to be followed)
        for (j, b), S in st_ref.items():
            ref = G.gla_step(*(t[b:b + 1, :, 0].float().cpu().numpy() for t in (gq, gk, gv, gg)), S)
            got = g_out[j][b, :, 0].float().cpu().numpy()
            assert (np.abs(got - ref[0]) <= 2e-2 + np.abs(ref[0]) * 2.0 ** -8).all(), f"{tag}: GLA layer {2 * j} row {b}"
        if deep:
            for j in sample_swa:
                for b in sample_b:
                    table, n, _ = views[b]
                    blocks = torch.tensor(table, device=dev)
                    kk = drv.kv_caches[j][0][blocks].float().cpu().numpy()
                    vv = drv.kv_caches[j][1][blocks].float().cpu().numpy()
                    ref = A.paged_decode_attention(q[b:b + 1].float().cpu().numpy(), kk, vv, np.arange(len(table))[None], [n],
                                                   D ** -0.5, WL)
                    assert np.abs(s_out[j][b:b + 1].float().cpu().numpy() - ref).max() <= 2e-2, f"{tag}: SWA layer {2 * j + 1} row {b}"

    # host-stepped steps (vectorised host manager, 256 rows)
    for step in range(3):
        fresh()
        meta = drv.step_metadata()
        layers(meta)
        torch.cuda.synchronize()
        check_step(meta.slot_mapping, meta.seq_lens_tensor, meta.block_tables, f"host step {step}", deep=step == 0)
    # device-side advance + all 28 layers in one captured graph
    drv.enable_device_advance()
    fresh()
    graph = drv.capture_step(layers)          # its warm-up pass is a real step on these inputs
    torch.cuda.synchronize()
    st = drv.device_state
    check_step(st.slot_mapping, st.seq_lens, st.block_tables, "capture warm-up step", deep=True)
    n_replays = 35
    for step in range(n_replays):
        fresh()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check_step(st.slot_mapping, st.seq_lens, st.block_tables, f"replay {step}", deep=step in (0, 15, 16, 17, n_replays - 1))
    st.check()
    # every byte of all 14 KV tensors after 39 steps
    for j in range(n_swa):
        assert torch.equal(drv.kv_caches[j], exp_kv[j]), f"SWA layer {2 * j + 1}: cache bytes"
    # sampled GLA states against the float64 recurrence
    for (j, b), S in st_ref.items():
        got = drv.gla_state[j, b].double().cpu().numpy()
        assert np.abs(got - S[0]).max() <= 1e-4 * np.abs(S[0]).max(), f"GLA layer {2 * j} row {b}: state"
    st.download()
    assert drv.manager.free_stack() == model.free
    # every sequence went through at least two block recycles
    assert all(((ctx[s] + 39) // BS) - (ctx[s] // BS) >= 2 for s in range(B))
