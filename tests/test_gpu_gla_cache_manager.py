"""`GLACacheManager(device="cuda")` driven the way the vLLM model drives it
(vllm_hymeta/model_for_7B/modeling_gla_swa.py:444-455 -> gla_cache.py:16-32 -> gla_attention.py:179-235):
per engine step `current_run_tensors` (request -> slot ids as a device tensor), `clear_prefill_slots` for
brand-new prompts, then per GLA layer the packed prompt kernel for the prefill rows and
`my_fused_recurrent_gla` for the decode rows on `GLACacheParams.at_layer_idx(i)`. The schedule covers a
sibling copy (parallel sampling), a finished request mapped to the pad slot in the step it finishes, slot
re-use by a new prompt in a mixed prefill + decode step, and a chunked prompt (context > 0: not cleared).
Every live slot's state in every layer is compared with the float64 oracle after every step (1e-4 of
the largest entry), outputs within 2e-2 + bf16 rounding; slots nobody owns must keep their fill."""
import numpy as np
import pytest
import torch

from oracle import gla as O

pytestmark = pytest.mark.gpu

LAYERS, SLOTS, H, D = 2, 5, 4, 128
SENTINEL = 12288.0   # exactly representable in bf16 too


class Engine:
    """Host model of the same schedule on numpy: slot ownership and float64 states per (layer, slot)."""

    def __init__(self, sb, dev, state_dtype):
        self.sb, self.dev = sb, dev
        self.mgr = sb.GLACacheManager(state_dtype, (LAYERS, SLOTS, H, D, D), device=dev)
        assert self.mgr.cache.is_cuda
        self.mgr.cache.fill_(SENTINEL)                       # stands for uninitialised memory (torch.empty)
        self.ref = np.full((LAYERS, SLOTS, H, D, D), SENTINEL, np.float64)
        self.g = torch.Generator().manual_seed(0)
        # a bf16 cache rounds the state once per call, when it is stored (my_fused_recurrent.py:79 stores in the
        # cache dtype; outputs come from the unrounded update): the model rounds at the same points
        self.bf16_state = state_dtype == torch.bfloat16
        self.state_tol = 1e-4 if state_dtype == torch.float32 else 2.0 ** -8

    def stored(self, x):
        return torch.from_numpy(x).bfloat16().double().numpy() if self.bf16_state else x

    def draw(self, n):
        q, k, v = (torch.randn(LAYERS, n, H, D, generator=self.g).bfloat16() for _ in range(3))
        gk = torch.nn.functional.logsigmoid(torch.randn(LAYERS, n, H, D, generator=self.g)) / 16
        return q, k, v, gk

    def step(self, prefills, decodes, finished=(), expect_slots=None):
        """prefills: [(request, seq, n_tokens, context_len)], decodes: [(request, seq)] in batch order
        (prefills first, as the backend lays tokens out); finished: request ids that ended."""
        sb, dev = self.sb, self.dev
        r2s = {}
        for req, seq, *_ in list(prefills) + list(decodes):
            r2s.setdefault(req, []).append(seq)
        cache, idx = self.mgr.current_run_tensors(request_ids_to_seq_ids=r2s, finished_requests_ids=list(finished))
        assert idx.is_cuda and idx.dtype == torch.int32 and cache is self.mgr.cache
        # current_run_tensors orders slots by request then sequence: map them back to (request, seq)
        flat = [(req, seq) for req, seqs in r2s.items() for seq in seqs]
        slot_of = dict(zip(flat, idx.tolist()))
        if expect_slots is not None:
            assert [slot_of[(r, s)] for r, s, *_ in list(prefills) + list(decodes)] == expect_slots
        from spikingbrain_7b_amd.gla import clear_prefill_slots
        ctx = [c for *_, c in prefills]
        # the model hands over request_ids_to_seq_ids in batch order; build that order explicitly
        order = {}
        for req, seq, *_ in list(prefills) + list(decodes):
            order.setdefault(req, []).append(seq)
        cleared = clear_prefill_slots(self.mgr, len(prefills), ctx, order)
        for (req, seq, n, c) in prefills:
            if c == 0 and slot_of[(req, seq)] >= 0:
                assert slot_of[(req, seq)] in cleared
                self.ref[:, slot_of[(req, seq)]] = 0.0
        n_pre = sum(n for _, _, n, _ in prefills)
        n_tok = n_pre + len(decodes)
        q, k, v, gk = self.draw(n_tok)
        batch_slots = [slot_of[(r, s)] for r, s, *_ in list(prefills) + list(decodes)]
        slots_dev = torch.tensor(batch_slots, dtype=torch.int32, device=dev)
        cu = np.cumsum([0] + [n for _, _, n, _ in prefills]).astype(np.int32)
        params = sb.GLACacheParams(cache, slots_dev)
        for layer in range(LAYERS):
            p = params.at_layer_idx(layer)
            assert p.gla_cache.data_ptr() == cache[layer].data_ptr()
            ql, kl, vl, gl = (t[layer].to(dev) for t in (q, k, v, gk))
            if prefills:
                o_pre = sb.gla_prefill_packed(ql, kl, vl, gl, p.gla_cache, p.state_indices_tensor,
                                              torch.from_numpy(cu).to(dev), len(prefills), max(n for _, _, n, _ in prefills))
                for i, (req, seq, n, c) in enumerate(prefills):
                    s = batch_slots[i]
                    sl = slice(cu[i], cu[i + 1])
                    args = [t[layer, sl].float().numpy().transpose(1, 0, 2)[None] for t in (q, k, v, gk)]   # [1, H, T, D]
                    o_ref, S = O.gla_recurrent(*args, initial_state=self.ref[layer, s][None])
                    self.ref[layer, s] = self.stored(S[0])
                    got = o_pre[sl].float().cpu().numpy().transpose(1, 0, 2)
                    tol = 2e-2 + 2.0 ** -8 * np.abs(o_ref[0]) + 2.0 ** -9 * np.abs(o_ref[0]).max()
                    assert (np.abs(got - o_ref[0]) <= tol).all()
            if decodes:
                dq, dk, dv, dg = (t[n_pre:].unsqueeze(2).contiguous() for t in (ql, kl, vl, gl))  # [B, H, 1, D]
                dslots = p.state_indices_tensor[len(prefills):]
                o = sb.my_fused_recurrent_gla(dq, dk, dv, dg, p.gla_cache, dslots)
                ds = batch_slots[len(prefills):]
                o_ref = O.gla_step(*(t[layer, n_pre:].float().numpy() for t in (q, k, v, gk)), self.ref[layer], slot_idx=ds)
                got = o.float().cpu().numpy()
                for s in ds:
                    if s >= 0:
                        self.ref[layer, s] = self.stored(self.ref[layer, s])
                for b, s in enumerate(ds):
                    if s < 0:
                        assert (got[b] == 0).all()          # pad-slot rows are skipped (output buffer starts zeroed)
                    else:
                        assert (np.abs(got[b] - o_ref[b]) <= 2e-2 + 2.0 ** -8 * np.abs(o_ref[b])).all()
        torch.cuda.synchronize()
        self.check()
        return slot_of

    def copy_slot(self, src, dst):
        self.ref[:, dst] = self.ref[:, src]

    def check(self):
        got = self.mgr.cache.double().cpu().numpy()
        for layer in range(LAYERS):
            for s in range(SLOTS):
                ref = self.ref[layer, s]
                if (ref == SENTINEL).all():
                    assert (got[layer, s] == SENTINEL).all(), f"slot {s} of layer {layer} was touched"
                else:
                    assert np.abs(got[layer, s] - ref).max() <= self.state_tol * max(np.abs(ref).max(), 1e-30)


@pytest.mark.parametrize("state_dtype", [torch.float32, torch.bfloat16])
def test_manager_schedule_on_device(sb, dev, state_dtype):
    e = Engine(sb, dev, state_dtype)
    # 1. two new prompts (one long enough for the matrix-core prompt kernel, one short): highest free slot first
    e.step(prefills=[("a", 0, 40, 0), ("b", 1, 7, 0)], decodes=[], expect_slots=[4, 3])
    # 2. both decode
    e.step(prefills=[], decodes=[("a", 0), ("b", 1)], expect_slots=[4, 3])
    # 3. request a forks a second sequence (parallel sampling): its slot starts as a copy of a's state in every layer
    e.copy_slot(4, 2)
    e.step(prefills=[], decodes=[("a", 0), ("a", 5), ("b", 1)], expect_slots=[4, 2, 3])
    # 4. b finishes: in this step its row maps to the pad slot (skipped), its slot goes back to the free stack
    slots = e.step(prefills=[], decodes=[("a", 0), ("a", 5), ("b", 1)], finished=["b"], expect_slots=[4, 2, -1])
    assert slots[("b", 1)] == sb.PAD_SLOT_ID
    # 5. mixed step: new prompt c takes b's old slot (cleared: it still holds b's state), a's sequences decode
    e.step(prefills=[("c", 9, 33, 0)], decodes=[("a", 0), ("a", 5)], expect_slots=[3, 4, 2])
    # 6. second chunk of c's prompt (context 33 > 0: the slot must NOT be cleared), a decodes on
    e.step(prefills=[("c", 9, 20, 33)], decodes=[("a", 0), ("a", 5)], expect_slots=[3, 4, 2])
    # 7. a finishes (both sequences), c decodes; slots 0 and 1 were never used
    e.step(prefills=[], decodes=[("c", 9)], finished=["a"], expect_slots=[3])
    assert sorted(e.mgr.free_cache_indices) == [0, 1, 2, 4]
    assert (e.mgr.cache[:, :2] == SENTINEL).all()


def test_capture_inputs_and_copy_before_graphs_on_device(sb, dev):
    """The graph-capture side of the manager (gla_cache.py via ConstantSizeCache): the padded slot buffer lives
    on the device, pad rows are -1, and a decode launch over the padded batch touches only the live slots."""
    m = sb.GLACacheManager(torch.float32, (1, 4, H, D, D), device=dev)
    m.cache.zero_()
    cache, buf = m.get_seqlen_agnostic_capture_inputs(6)
    assert buf.is_cuda and buf.tolist() == [sb.PAD_SLOT_ID] * 6
    m.copy_inputs_before_cuda_graphs({"seqlen_agnostic_capture_inputs": (cache, buf)},
                                     request_ids_to_seq_ids={"x": [0], "y": [1]}, finished_requests_ids=[])
    torch.cuda.synchronize()
    assert buf.tolist() == [3, 2, -1, -1, -1, -1]
    same = m.current_run_tensors(seqlen_agnostic_capture_inputs=(cache, buf))
    assert same[0] is cache and same[1] is buf
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(6, H, 1, D, generator=g).bfloat16().to(dev) for _ in range(3))
    gk = (torch.nn.functional.logsigmoid(torch.randn(6, H, 1, D, generator=g)) / 16).to(dev)
    o = sb.my_fused_recurrent_gla(q, k, v, gk, cache[0], buf)
    ref_state = np.zeros((4, H, D, D))
    o_ref = O.gla_step(*(t[:, :, 0].float().cpu().numpy() for t in (q, k, v, gk)), ref_state, slot_idx=buf.tolist())
    got = o.float().cpu().numpy()
    assert (got[2:] == 0).all() and (np.abs(got[:2] - o_ref[:2]) <= 2e-2 + 2.0 ** -8 * np.abs(o_ref[:2])).all()
    st = cache[0].double().cpu().numpy()
    assert (st[:2] == 0).all() and np.abs(st[2:] - ref_state[2:]).max() <= 1e-4 * np.abs(ref_state).max()
