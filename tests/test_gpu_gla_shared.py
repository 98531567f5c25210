"""Shared GLA states: k, v and the gate come with the 4 kv heads, as the model computes them before its
repeat_kv (hf_7B_model/gla_attention.py:147-149), and one state per kv head serves its 7 query heads.
Checked against (1) the oracle run the reference's way, on repeated k, v, g with 28 states, and (2) this
library's own one-state-per-head kernels on the repeated tensors, which every shared-state kernel must
reproduce bit for bit (same update and summation order)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gla as G

pytestmark = pytest.mark.gpu

D = 128
STATE_RTOL = 1e-4
OUT_ATOL = 2e-2


def make(B, H, Hk, T, seed, dtype=torch.bfloat16, relu=False):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, T, D, generator=g).to(dtype)
    k, v = (torch.randn(B, Hk, T, D, generator=g).to(dtype) for _ in range(2))
    if relu:  # the model's activation on q and k (hf_7B_model/gla_attention.py:134-135)
        q, k = q.relu(), k.relu()
    gate = F.logsigmoid(torch.randn(B, Hk, T, D, generator=g)) / 16
    return q, k, v, gate


def rep(x, n):
    return x.repeat_interleave(n, dim=1)


def close(got, ref, block_form=False):
    """2e-2 max-abs on the fp32 result plus the rounding of the stored bf16 output (half an ulp, 2^-8
    relative). The matrix-core block form also rounds the operands of q.S to bf16, like any bf16 GEMM (and
    like the chunked kernel the reference prefills with): that error follows the size of the summed terms,
    not of the result, so it is bounded against the largest output of the call (2^-9 of it; measured up
    to 0.05 on outputs near 3 where the largest is 36)."""
    tol = OUT_ATOL + 2.0 ** -8 * np.abs(ref) + (2.0 ** -9 * np.abs(ref).max() if block_form else 0.0)
    return bool((np.abs(got - ref) <= tol).all())


@pytest.mark.parametrize("state_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,H,Hk,T", [(5, 28, 4, 1), (3, 28, 4, 3), (2, 16, 2, 1), (4, 8, 4, 2), (2, 6, 1, 1)])
def test_decode_shared_vs_oracle_and_per_head_kernel(sb, dev, state_dtype, B, H, Hk, T):
    n = H // Hk
    q, k, v, gate = make(B, H, Hk, T, 100 * B + H + T)
    g = torch.Generator().manual_seed(5)
    slots = B + 3
    state = (torch.randn(slots, Hk, D, D, generator=g) * 0.02).to(state_dtype)
    slot_idx = torch.randperm(slots, generator=g)[:B].to(torch.int32)
    if B > 2:
        slot_idx[1] = -1
    live = [b for b in range(B) if slot_idx[b] >= 0]
    live_slots = [int(slot_idx[b]) for b in live]

    # the reference's layout: 28 states, repeated k, v, g
    ref_state = rep(state, n).double().numpy().copy()
    ref_o = np.zeros((B, H, T, D))
    for t in range(T):
        ref_o[:, :, t] = G.gla_step(q[:, :, t].float().numpy(), rep(k, n)[:, :, t].float().numpy(),
                                    rep(v, n)[:, :, t].float().numpy(), rep(gate, n)[:, :, t].numpy(),
                                    ref_state, slot_idx.tolist())
    # the heads of a group end with identical states
    assert np.array_equal(ref_state.reshape(slots, Hk, n, D, D), np.repeat(ref_state[:, ::n, None], n, 2))

    st = state.to(dev)
    out = torch.zeros(B, H, T, D, dtype=q.dtype, device=dev)
    sb.ops.gla_recurrent(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st, slot_idx.to(dev), out=out)
    st_full = rep(state, n).contiguous().to(dev)
    out_full = torch.zeros_like(out)
    sb.ops.gla_recurrent(q.to(dev), rep(k, n).to(dev), rep(v, n).to(dev), rep(gate, n).to(dev), st_full,
                         slot_idx.to(dev), out=out_full)
    torch.cuda.synchronize()

    assert torch.equal(out, out_full)
    assert torch.equal(st, st_full[:, ::n])
    got_state = st.double().cpu().numpy()
    tol = STATE_RTOL if state_dtype == torch.float32 else 2 ** -8 * T
    err = np.abs(got_state[live_slots] - ref_state[live_slots][:, ::n]).max() / np.abs(ref_state[live_slots]).max()
    assert err <= tol
    assert close(out.float().cpu().numpy()[live], ref_o[live])
    dead = sorted(set(range(slots)) - set(live_slots))
    assert torch.equal(st.cpu()[dead], state[dead])
    if len(live) < B:
        assert not out[1].any()


@pytest.mark.parametrize("per_head", [True, False])
@pytest.mark.parametrize("dtype,T", [(torch.bfloat16, 8), (torch.bfloat16, 40), (torch.bfloat16, 100),
                                      (torch.float32, 21), (torch.float16, 9)])
def test_prompt_shared_states_start_from_live_state(sb, dev, dtype, T, per_head):
    """Many-step calls (the step-by-step kernel for short or non-bf16 calls, the matrix-core block form
    from 32 steps on): every head of a group must see the state as it was BEFORE the call, although the
    group's first head overwrites it. The block form in both of its shapes: one workgroup per query head
    (two ordered launches) and one per group of query heads (the state advanced once)."""
    B, H, Hk = 3, 28, 4
    n = H // Hk
    q, k, v, gate = make(B, H, Hk, T, T, dtype, relu=True)
    g = torch.Generator().manual_seed(11)
    state = torch.randn(B, Hk, D, D, generator=g) * 0.02
    ref_o, ref_S = G.gla_recurrent(q.float().numpy(), rep(k, n).float().numpy(), rep(v, n).float().numpy(),
                                   rep(gate, n).numpy(), rep(state, n).double().numpy())
    st = state.to(dev)
    out = sb.ops.gla_recurrent(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st, per_head=per_head)
    st_full = rep(state, n).contiguous().to(dev)
    out_full = sb.ops.gla_recurrent(q.to(dev), rep(k, n).to(dev), rep(v, n).to(dev), rep(gate, n).to(dev), st_full)
    torch.cuda.synchronize()
    assert torch.equal(out, out_full)
    assert torch.equal(st, st_full[:, ::n])
    assert np.abs(st.double().cpu().numpy() - ref_S[:, ::n]).max() / np.abs(ref_S).max() <= STATE_RTOL
    if dtype == torch.float32:
        assert np.abs(out.double().cpu().numpy() - ref_o).max() <= 1e-4 * max(1.0, np.abs(ref_o).max())
    else:
        assert close(out.float().cpu().numpy(), ref_o, block_form=T >= 32)


@pytest.mark.parametrize("per_head,H,Hk,gdtype,sdtype", [(True, 28, 4, torch.float32, torch.float32),
                                                          (False, 28, 4, torch.float32, torch.float32),
                                                          (False, 16, 2, torch.bfloat16, torch.bfloat16),
                                                          (False, 6, 3, torch.float16, torch.float32),
                                                          (None, 28, 4, torch.float32, torch.float32)])
def test_packed_prompts_shared_states(sb, dev, per_head, H, Hk, gdtype, sdtype):
    n = H // Hk
    lens = [5, 70, 1, 33, 16]
    total = sum(lens)
    g = torch.Generator().manual_seed(3)
    q = torch.randn(total, H, D, generator=g).bfloat16().relu()
    k = torch.randn(total, Hk, D, generator=g).bfloat16().relu()
    v = torch.randn(total, Hk, D, generator=g).bfloat16()
    gate = (F.logsigmoid(torch.randn(total, Hk, D, generator=g)) / 16).to(gdtype)
    slots = 8
    state = (torch.randn(slots, Hk, D, D, generator=g) * 0.02).to(sdtype)
    slot_idx = torch.tensor([6, 0, -1, 3, 5], dtype=torch.int32)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)

    st = state.to(dev)
    out = torch.zeros(total, H, D, dtype=torch.bfloat16, device=dev)
    sb.ops.gla_recurrent_packed(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st, cu.to(dev), slot_idx.to(dev),
                                out=out, max_seq_len=max(lens), per_head=per_head)
    st_full = rep(state, n).contiguous().to(dev)
    out_full = torch.zeros_like(out)
    sb.ops.gla_recurrent_packed(q.to(dev), rep(k, n).to(dev), rep(v, n).to(dev), rep(gate, n).to(dev), st_full,
                                cu.to(dev), slot_idx.to(dev), out=out_full, max_seq_len=max(lens))
    torch.cuda.synchronize()
    assert torch.equal(out, out_full)
    assert torch.equal(st, st_full[:, ::n])
    # and against the oracle, sequence by sequence
    for i, L in enumerate(lens):
        s = int(slot_idx[i])
        sl = slice(int(cu[i]), int(cu[i + 1]))
        if s < 0:
            assert not out[sl].any()
            continue
        tr = lambda x: x[sl].transpose(0, 1)[None]  # [1, heads, L, D]
        ref_o, ref_S = G.gla_recurrent(tr(q).float().numpy(), rep(tr(k), n).float().numpy(),
                                       rep(tr(v), n).float().numpy(), rep(tr(gate), n).float().numpy(),
                                       rep(state[s][None], n).double().numpy())
        assert close(out[sl].float().cpu().numpy(), ref_o[0].transpose(1, 0, 2), block_form=True)
        rtol = STATE_RTOL if sdtype == torch.float32 else 2.0 ** -8          # (a bf16 state cache rounds what it stores)
        assert np.abs(st[s].double().cpu().numpy() - ref_S[0, ::n]).max() / np.abs(ref_S).max() <= rtol
    assert torch.equal(st.cpu()[[1, 2, 4, 7]], state[[1, 2, 4, 7]])


def test_reference_named_wrappers_take_kv_heads(sb, dev):
    B, H, Hk = 4, 28, 4
    q, k, v, gate = make(B, H, Hk, 1, 77)
    cache = torch.zeros(6, Hk, D, D, device=dev)
    slots = torch.tensor([2, 0, 5, 1], dtype=torch.int32, device=dev)
    o = sb.my_fused_recurrent_gla(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), cache, slots)
    full = torch.zeros(6, H, D, D, device=dev)
    o_full = sb.my_fused_recurrent_gla(q.to(dev), rep(k, 7).to(dev), rep(v, 7).to(dev), rep(gate, 7).to(dev), full, slots)
    assert o.shape == (B, H, D) and torch.equal(o, o_full) and torch.equal(cache, full[:, ::7])
    q2, k2, v2, g2 = make(2, H, Hk, 48, 78)
    o2, S2 = sb.fused_chunk_gla(q2.to(dev), k2.to(dev), v2.to(dev), g2.to(dev), output_final_state=True)
    o2f, S2f = sb.fused_chunk_gla(q2.to(dev), rep(k2, 7).to(dev), rep(v2, 7).to(dev), rep(g2, 7).to(dev),
                                  output_final_state=True)
    assert S2.shape == (2, Hk, D, D) and torch.equal(o2, o2f) and torch.equal(S2, S2f[:, ::7])


def test_shared_state_argument_errors(sb, dev):
    q, k, v, gate = make(1, 28, 4, 1, 1)
    with pytest.raises(ValueError):   # 28 query heads over 5 kv heads
        sb.ops.gla_recurrent(q.to(dev), torch.zeros(1, 5, 1, D, dtype=q.dtype, device=dev),
                             torch.zeros(1, 5, 1, D, dtype=q.dtype, device=dev), torch.zeros(1, 5, 1, D, device=dev),
                             torch.zeros(1, 5, D, D, device=dev))
    with pytest.raises(ValueError):   # state must have the kv heads
        sb.ops.gla_recurrent(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), torch.zeros(1, 28, D, D, device=dev))
    with pytest.raises(ValueError):   # more than 8 query heads per state
        sb.ops.gla_recurrent(torch.zeros(1, 18, 1, D, dtype=q.dtype, device=dev), k[:, :2].to(dev), v[:, :2].to(dev),
                             gate[:, :2].to(dev), torch.zeros(1, 2, D, D, device=dev))
