"""Device-side decode-step advance (sb_window_advance) against the host block manager and the
brute-force oracle model: slots, visible lengths, block-table rows and the free-stack order must
be identical, step after step, for aligned and unaligned windows, staggered sequence lengths
(so evictions and allocations fall on different steps) and a nearly empty free stack."""
import copy

import numpy as np
import pytest
import torch

from oracle import paged as P

pytestmark = pytest.mark.gpu


def make(sb, bs, wl, prompts, nb):
    mgr = sb.WindowBlockManager(nb, bs, wl, max_seqs=len(prompts), max_chunk_tokens=max(prompts) + 1)
    model = P.WindowCacheModel(nb, bs, wl)
    for s, n in enumerate(prompts):
        mgr.add_seq(s); model.add_seq(s)
        a = mgr.append_tokens(s, n, True)
        b = model.append_tokens(s, n, True)
        assert a == b
    return mgr, model


@pytest.mark.parametrize("bs,wl", [(16, 64), (16, 40), (32, 100), (16, 0)])
def test_device_advance_matches_host_and_oracle(sb, dev, bs, wl):
    prompts = [1, 15, 16, 17, 63, 64, 65, 200, 1000, 1001, 5, 333]
    nb = sum((min(n, wl + 1) + bs - 1) // bs + 2 for n in prompts) + 3
    mgr, model = make(sb, bs, wl, prompts, nb)
    host = copy.deepcopy(mgr)
    seqs = list(range(len(prompts)))
    state = sb.block_manager.DeviceWindowState(mgr, seqs, dev)
    W = state.table_width
    for step in range(3 * bs + 5):
        state.advance()
        slots = host.decode_step(seqs)
        tables, lens, _ = host.kernel_view(seqs, pad_blocks=W)
        ref_slots = [model.append_tokens(s, 1, False)[0] for s in seqs]
        assert slots.tolist() == ref_slots
        assert state.slot_mapping.cpu().tolist() == ref_slots, f"step {step}"
        assert state.seq_lens.cpu().tolist() == lens.tolist()
        assert np.array_equal(state.block_tables.cpu().numpy(), tables)
        for s in seqs:
            t, n, _ = model.view(s)
            assert tables[s, :len(t)].tolist() == t and n == lens[s]
    state.download()          # also checks the status word
    assert mgr.free_stack() == host.free_stack() == model.free
    assert np.array_equal(mgr.n_tokens, host.n_tokens)
    assert np.array_equal(mgr.lo, host.lo) and np.array_equal(mgr.hi, host.hi)
    for s in seqs:            # ring entries of resident blocks
        for j in range(int(host.lo[s]), int(host.hi[s]) + 1):
            assert mgr.ring[s, j % mgr.ring_blocks] == host.ring[s, j % host.ring_blocks]


def test_device_advance_large_aligned_batch(sb, dev):
    """The serving shape in small: every sequence window-saturated at the same length, so all of them
    recycle a block on the same step (push followed by pop, in row order)."""
    B, bs, wl = 300, 16, 128
    mgr = sb.WindowBlockManager(B * (wl // bs + 2) + 4, bs, wl, max_seqs=B)
    for s in range(B):
        mgr.add_seq(s)
        mgr.append_tokens(s, 100000, True)
    host = copy.deepcopy(mgr)
    state = sb.block_manager.DeviceWindowState(mgr, list(range(B)), dev)
    for step in range(2 * bs + 1):
        state.advance()
        slots = host.decode_step(list(range(B)))
        assert state.slot_mapping.cpu().tolist() == slots.tolist(), f"step {step}"
    tables, lens, _ = host.kernel_view(list(range(B)), pad_blocks=state.table_width)
    assert np.array_equal(state.block_tables.cpu().numpy(), tables)
    assert state.seq_lens.cpu().tolist() == lens.tolist()
    state.download()
    assert mgr.free_stack() == host.free_stack()


def test_device_advance_reports_exhaustion(sb, dev):
    bs, wl = 16, 64
    mgr = sb.WindowBlockManager(1, bs, wl, max_seqs=1)      # one block in total
    mgr.add_seq(0)
    mgr.append_tokens(0, 16, True)                           # takes it
    state = sb.block_manager.DeviceWindowState(mgr, [0], dev)
    state.advance()                                          # token 16 needs a second block
    with pytest.raises(RuntimeError, match="out of KV cache blocks"):
        state.check()


def test_exhaustion_touches_no_foreign_block(sb, dev):
    """Free stack empty while one sequence must grow into a new block: that row gets the pad slot (its append
    is skipped), keeps its token count and length, and the other sequences' blocks, slots and cache rows are
    what they would be anyway. The host manager raises at the same point; the device reports through status."""
    bs, wl, Hkv, D = 16, 64, 4, 128
    mgr = sb.WindowBlockManager(3, bs, wl, max_seqs=2)       # three blocks in total
    mgr.add_seq(0); mgr.add_seq(1)
    mgr.append_tokens(0, 16, True)                           # block 0 full: the next token needs a new block
    mgr.append_tokens(1, 20, True)                           # two blocks, room in the second
    assert mgr.num_free_blocks == 0
    before = dict(tok=mgr.n_tokens[:2].copy(), ring=mgr.ring[:2].copy())
    state = sb.block_manager.DeviceWindowState(mgr, [0, 1], dev)
    kv = torch.zeros(2, 3, bs, Hkv, D, dtype=torch.bfloat16, device=dev)
    for step in range(2):                                    # the failing row fails again on the next step
        state.advance()
        torch.cuda.synchronize()
        assert state.slot_mapping.tolist()[0] == sb.PAD_SLOT_ID
        assert state.n_tokens.tolist() == [16, 21 + step] and state.seq_lens.tolist() == [16, 21 + step]
        assert np.array_equal(state.ring.cpu().numpy(), before["ring"])           # no id handed out, none overwritten
        pos = 20 + step
        assert state.slot_mapping.tolist()[1] == int(before["ring"][1][pos // bs]) * bs + pos % bs
        assert state.block_tables[0].tolist()[:1] == [int(before["ring"][0][0])]
        k = torch.full((2, Hkv, D), float(step + 1), dtype=torch.bfloat16, device=dev)
        sb.ops.kv_append(k, k, kv[0], kv[1], state.slot_mapping)
        torch.cuda.synchronize()
        written = (kv[0] != 0).flatten(2).any(2).nonzero().tolist()               # (block, row) pairs holding data
        assert written == [[int(before["ring"][1][1]), 4 + s] for s in range(step + 1)]
    with pytest.raises(RuntimeError, match="out of KV cache blocks"):
        state.check()
