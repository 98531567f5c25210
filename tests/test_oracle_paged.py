"""Pins oracle.paged (append, slot mapping, the window block-manager model) by brute force, then
checks the product's vectorised WindowBlockManager against that model bit for bit."""
import numpy as np
import pytest

from oracle import paged as P


def test_kv_append_closed_form_and_sentinels():
    r = np.random.default_rng(0)
    nb, bs, H, D, T = 6, 16, 2, 4, 9
    kc = np.full((nb, bs, H, D), -7.0); vc = np.full((nb, bs, H, D), -9.0)
    key = r.standard_normal((T, H, D)); val = r.standard_normal((T, H, D))
    slots = [5, 16, -1, 95, 0, 17, -1, 40, 41]
    P.kv_append(key, val, kc, vc, slots)
    flat_k = kc.reshape(nb * bs, H, D); flat_v = vc.reshape(nb * bs, H, D)
    written = [s for s in slots if s >= 0]
    for t, s in enumerate(slots):
        if s >= 0:
            assert np.array_equal(flat_k[s], key[t]) and np.array_equal(flat_v[s], val[t])
    untouched = np.setdiff1d(np.arange(nb * bs), written)
    assert (flat_k[untouched] == -7.0).all() and (flat_v[untouched] == -9.0).all()


def test_slot_mapping_functions():
    assert P.compute_slot_mapping_start_idx(True, 100, 0, 32) == 68
    assert P.compute_slot_mapping_start_idx(True, 10, 0, 32) == 0
    assert P.compute_slot_mapping_start_idx(False, 1, 500, 32) == 0      # decode: never skipped
    assert P.compute_slot_mapping_start_idx(True, 100, 0, None) == 0
    bt = {7: [9, 3, 5]}
    out = []
    P.compute_slot_mapping(False, out, 7, 40, 0, 20, 16, bt)             # tokens 0..19 PAD, 20..39 mapped
    assert out[:20] == [-1] * 20
    assert out[20:] == [bt[7][i // 16] * 16 + i % 16 for i in range(20, 40)]
    out = []
    P.compute_slot_mapping(False, out, 7, 41, 40, 0, 16, bt)             # one decode token at position 40
    assert out == [5 * 16 + 8]
    out = []
    P.compute_slot_mapping(True, out, 7, 5, 0, 0, 16, bt)                # profile run: all PAD
    assert out == [-1] * 5


@pytest.mark.parametrize("bs,wl", [(16, 32), (16, 40), (32, 64), (16, 0)])
def test_model_residency_invariant_brute_force(bs, wl):
    """After every token: every position a query at the newest position may see is resident, at
    the slot the closed form gives, and nothing older than one block before the window is kept."""
    m = P.WindowCacheModel(64, bs, wl)
    m.add_seq(0)
    where = {}                                   # absolute position -> slot, filled from returned slots
    prompt = 3 * wl // 2 + 7
    slots = m.append_tokens(0, prompt, True)
    assert slots[:max(0, prompt - wl)] == [-1] * max(0, prompt - wl)
    for i, s in enumerate(slots):
        if s >= 0:
            where[i] = s
    n = prompt
    for step in range(5 * bs + 3):
        (s,) = m.append_tokens(0, 1, False)
        where[n] = s
        n += 1
        table, seqlen, first = m.view(0)
        p = n - 1
        assert first % bs == 0 and seqlen == n - first
        for pos in range(max(0, p - wl), p + 1):                         # the whole window is resident ...
            k = pos - first
            assert k >= 0
            assert table[k // bs] * bs + k % bs == where[pos]            # ... at the slot it was written to
        assert first >= max(0, (p - wl) // bs * bs - 0)                  # and no whole block before the window stays
        assert first <= max(0, p - wl)
        live = set(table)
        assert len(live) == len(table) and not live & set(m.free)        # no block both resident and free
    assert len(m.free) + len(m.view(0)[0]) == 64                         # nothing leaked


def test_model_recycles_own_block_when_window_is_block_aligned():
    m = P.WindowCacheModel(32, 16, 64)
    m.add_seq("a")
    m.append_tokens("a", 64, True)
    used = set()
    for _ in range(200):
        m.append_tokens("a", 1, False)
        used |= set(m.view("a")[0])
    assert len(used) == 64 // 16 + 1                                     # a fixed ring of wl/bs + 1 blocks


def run_schedule(mgr, model, seed, n_seqs, steps, bs, wl):
    r = np.random.default_rng(seed)
    live = []
    next_id = 0
    for step in range(steps):
        if len(live) < n_seqs and r.random() < 0.3:                      # a new prompt arrives
            sid = next_id; next_id += 1
            mgr.add_seq(sid); model.add_seq(sid)
            L = int(r.integers(1, 3 * wl + 5))
            chunks = [L] if r.random() < 0.5 else [L // 2, L - L // 2]
            for c in chunks:
                if c:
                    assert mgr.append_tokens(sid, c, True) == model.append_tokens(sid, c, True)
            live.append(sid)
        if live and r.random() < 0.1:
            sid = live.pop(int(r.integers(len(live))))
            mgr.free_seq(sid); model.free_seq(sid)
        if live:
            order = list(r.permutation(live))
            got = mgr.decode_step(order)
            exp = [model.append_tokens(s, 1, False)[0] for s in order]
            assert got.tolist() == exp
            tables, seqlens, first = mgr.kernel_view(order)
            for i, s in enumerate(order):
                t, n, f = model.view(s)
                assert tables[i, :len(t)].tolist() == t and (tables[i, len(t):] == 0).all()
                assert int(seqlens[i]) == n and int(first[i]) == f
        assert mgr.free_stack() == model.free


@pytest.mark.parametrize("seed,bs,wl", [(0, 16, 32), (1, 16, 48), (2, 32, 64), (3, 16, 40)])
def test_product_block_manager_matches_model(sb, seed, bs, wl):
    nb = 256
    mgr = sb.WindowBlockManager(nb, bs, wl, max_seqs=6, max_chunk_tokens=3 * wl + 5)
    model = P.WindowCacheModel(nb, bs, wl)
    run_schedule(mgr, model, seed, n_seqs=6, steps=120, bs=bs, wl=wl)


def test_product_slot_mapping_functions_match(sb):
    for args in [(True, 100, 0, 32), (True, 10, 0, 32), (False, 1, 500, 32), (True, 9, 4, None)]:
        assert sb.compute_slot_mapping_start_idx(*args) == P.compute_slot_mapping_start_idx(*args)
    bt = {0: list(range(50, 60))}
    for seq_len, ctx, start in [(40, 0, 20), (41, 40, 0), (100, 30, 50), (17, 16, 0)]:
        a, b = [], []
        sb.compute_slot_mapping(False, a, 0, seq_len, ctx, start, 16, bt)
        P.compute_slot_mapping(False, b, 0, seq_len, ctx, start, 16, bt)
        assert a == b
    a = []
    sb.compute_slot_mapping(True, a, 0, 5, 0, 0, 16, bt)
    assert a == [-1] * 5


def test_slot_buffer_path_matches_list_path(sb):
    """The builder's SlotBuffer (numpy pieces, vectorised table lookups through LogicalTable.blocks) gives the
    slots of the list path and of the oracle, sequence after sequence into one buffer; a lookup outside the
    resident range raises as the per-block path does."""
    from spikingbrain_7b_amd.block_manager import LogicalTable, SlotBuffer
    rng = np.random.default_rng(0)
    bs, wl = 16, 64
    mgr = sb.WindowBlockManager(512, bs, wl, max_seqs=4, max_chunk_tokens=400)
    buf, ref = SlotBuffer(), []
    for s in range(4):
        mgr.add_seq(s)
        n = int(rng.integers(1, 390))
        mgr.append_tokens(s, n, True, store_all=bool(s & 1), want_slots=False)
        r = mgr.row_of(s)
        start = P.compute_slot_mapping_start_idx(True, n, 0, None if s & 1 else wl)
        view = LogicalTable(mgr, r)
        sb.compute_slot_mapping(False, buf, r, n, 0, start, bs, {r: view})
        as_list = {r: {j: view[j] for j in range(int(mgr.lo[r]), int(mgr.hi[r]) + 1)}}
        P.compute_slot_mapping(False, ref, r, n, 0, start, bs, as_list)
        assert len(buf) == len(ref)
    assert buf.tolist() == ref and buf.array().dtype == np.int64
    buf.extend([-1] * 3)
    assert buf.tolist() == ref + [-1] * 3
    with pytest.raises(IndexError):
        LogicalTable(mgr, 0).blocks(int(mgr.hi[0]), int(mgr.hi[0]) + 1)
    empty = SlotBuffer()
    sb.compute_slot_mapping(True, empty, 0, 4, 0, 0, bs, None)
    assert empty.tolist() == [-1] * 4 and SlotBuffer().array().shape == (0,)


def test_block_manager_errors(sb):
    with pytest.raises(ValueError, match="multiple of 16"):
        sb.WindowBlockManager(8, 24, 32, max_seqs=1)
    m = sb.WindowBlockManager(2, 16, 64, max_seqs=1, max_chunk_tokens=64)
    m.add_seq(0)
    with pytest.raises(RuntimeError, match="out of KV cache blocks"):
        m.append_tokens(0, 64, True)
    with pytest.raises(KeyError):
        m.add_seq(0)


def _manager_state(m):
    return (m.free_stack(), m.ring.copy(), m.lo.copy(), m.hi.copy(), m.n_tokens.copy())


def _same_state(a, b):
    return a[0] == b[0] and all(np.array_equal(x, y) for x, y in zip(a[1:], b[1:]))


def test_exhausted_pool_leaves_the_manager_untouched(sb):
    """A step that runs out of blocks raises with nothing changed: no block is both free and resident, so
    freeing a sequence afterwards cannot hand one block to two sequences (prompt chunk with evictions,
    and a decode batch that fails at its second row)."""
    M = sb.block_manager.WindowBlockManager
    m = M(num_blocks=12, block_size=16, window_left=64, max_seqs=4, max_chunk_tokens=128)
    m.add_seq("a")
    m.add_seq("b")
    m.append_tokens("a", 96, True, store_all=True)      # 6 blocks
    m.append_tokens("b", 80, True, store_all=True)      # 5 blocks, 1 left
    before = _manager_state(m)
    with pytest.raises(RuntimeError, match="out of KV cache blocks"):
        m.append_tokens("a", 128, True, store_all=True)  # evicts 2, needs 8: 3 free in all
    assert _same_state(before, _manager_state(m))
    m.free_seq("a")
    free = m.free_stack()
    assert len(free) == len(set(free)) == 7
    resident_b = {int(m.ring[m.row_of("b"), j % m.ring_blocks]) for j in range(int(m.lo[m.row_of("b")]), int(m.hi[m.row_of("b")]) + 1)}
    assert not (resident_b & set(free))

    # decode batch: the first row's allocation succeeds on its own, the second finds the stack empty
    m = M(num_blocks=5, block_size=16, window_left=1024, max_seqs=4)
    for s in ("a", "b"):
        m.add_seq(s)
        m.append_tokens(s, 32, True)                     # 2 blocks each, both full: the next token allocates
    before = _manager_state(m)
    with pytest.raises(RuntimeError, match="out of KV cache blocks"):
        m.decode_step(["a", "b"])
    assert _same_state(before, _manager_state(m))
    m.free_seq("b")
    slots = m.decode_step(["a"])
    assert slots.shape == (1,) and len(set(m.free_stack())) == m.num_free_blocks == 2
