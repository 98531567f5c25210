"""GLA recurrent kernel vs the float64 oracle. Tolerances (BASELINE): state 1e-4 relative to
the largest state entry, output 2e-2 max-abs for bf16 q/k/v."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gla as G

pytestmark = pytest.mark.gpu

STATE_RTOL = 1e-4
OUT_ATOL = 2e-2


def out_close(got, ref, dtype=torch.bfloat16):
    """max-abs 2e-2 on the fp32 result; storing it in bf16 adds at most half a bf16 ulp
    (up to 2^-8 relative: 7 stored mantissa bits), more than 2e-2 once |o| > 5, so that rounding
    is allowed on top."""
    half_ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 0.0}[dtype]
    return bool((np.abs(got - ref) <= OUT_ATOL + half_ulp * np.abs(ref)).all())


def make(B, H, T, D, seed, dtype=torch.bfloat16, relu=False):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(B, H, T, D, generator=g).to(dtype) for _ in range(3))
    if relu:
        q, k = q.relu(), k.relu()
    gate = F.logsigmoid(torch.randn(B, H, T, D, generator=g)) / 16
    return q, k, v, gate


def rel(a, b):
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


@pytest.mark.parametrize("state_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,H,slots", [(5, 28, 9), (1, 4, 1), (64, 7, 64)])
def test_decode_step_vs_oracle(sb, dev, state_dtype, B, H, slots):
    D = 128
    q, k, v, gate = make(B, H, 1, D, B * 31 + H)
    g = torch.Generator().manual_seed(7)
    state = (torch.randn(slots, H, D, D, generator=g) * 0.02).to(state_dtype)
    slot_idx = torch.randperm(slots, generator=g)[:B].to(torch.int32)
    if B > 2:
        slot_idx[1] = -1
    ref_state = state.double().numpy().copy()
    ref_o = G.gla_step(q[:, :, 0].float().numpy(), k[:, :, 0].float().numpy(), v[:, :, 0].float().numpy(),
                       gate[:, :, 0].numpy(), ref_state, slot_idx.tolist())
    st = state.to(dev)
    o = sb.my_fused_recurrent_gla(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st, slot_idx.to(dev))
    torch.cuda.synchronize()
    assert o.shape == (B, H, D) and o.dtype == q.dtype
    got_state = st.double().cpu().numpy()
    live = [b for b in range(B) if slot_idx[b] >= 0]
    skipped_slots = sorted(set(range(slots)) - {int(slot_idx[b]) for b in live})
    tol = STATE_RTOL if state_dtype == torch.float32 else 2 ** -8   # bf16 storage rounds to 8 bits
    assert rel(got_state[[int(slot_idx[b]) for b in live]], ref_state[[int(slot_idx[b]) for b in live]]) <= tol
    # untouched slots are bit-identical
    assert np.array_equal(got_state[skipped_slots], state.double().numpy()[skipped_slots])
    assert out_close(o.float().cpu().numpy()[live], ref_o[live])
    if B > 2:
        assert (o[1] == 0).all()        # skipped row: output buffer left as allocated (zeros)


def test_special_cases_on_device(sb, dev):
    B, H, D = 2, 3, 128
    q, k, v, gate = make(B, H, 1, D, 5, dtype=torch.float32)
    S0 = torch.randn(B, H, D, D) * 0.1
    # k = 0, g = 0 leaves the state bit-identical and o = scale * q S
    st = S0.clone().to(dev)
    o = sb.my_fused_recurrent_gla(q.to(dev), torch.zeros_like(k).to(dev), v.to(dev), torch.zeros_like(gate).to(dev), st, None, scale=0.5)
    assert torch.equal(st.cpu(), S0)
    np.testing.assert_allclose(o.cpu().numpy(), 0.5 * torch.einsum("bhk,bhkv->bhv", q[:, :, 0], S0).numpy(), rtol=1e-4, atol=1e-5)
    # q = e_i / scale reads row i of the updated state exactly
    e = torch.zeros(B, H, 1, D); e[..., 5] = 4.0
    st = S0.clone().to(dev)
    o = sb.my_fused_recurrent_gla(e.to(dev), k.to(dev), v.to(dev), gate.to(dev), st, None, scale=0.25)
    assert torch.equal(o.cpu(), st.cpu()[:, :, 5, :])


@pytest.mark.parametrize("T", [1, 2, 17])
def test_multi_step_vs_oracle_and_layouts(sb, dev, T):
    B, H, D = 3, 4, 128
    q, k, v, gate = make(B, H, T, D, 11 + T, relu=True)
    S0 = torch.randn(B, H, D, D) * 0.02
    ref_o, ref_S = G.gla_recurrent(q.float().numpy(), k.float().numpy(), v.float().numpy(), gate.numpy(), S0.numpy())
    # head-first views of token-major projections, as the HF layer produces them
    qd, kd, vd, gd = (x.transpose(1, 2).contiguous().to(dev).transpose(1, 2) for x in (q, k, v, gate))
    o, S = sb.fused_recurrent_gla(qd, kd, vd, gd, initial_state=S0.to(dev), output_final_state=True)
    assert rel(S.double().cpu().numpy(), ref_S) <= STATE_RTOL
    assert out_close(o.float().cpu().numpy(), ref_o)
    # stepping T times with T=1 gives the same state as one call with T steps (same fp32 op order)
    st = S0.clone().to(dev)
    for t in range(T):
        sb.fused_recurrent_gla(qd[:, :, t:t + 1], kd[:, :, t:t + 1], vd[:, :, t:t + 1], gd[:, :, t:t + 1],
                               initial_state=st, output_final_state=True, inplace_state=True)
    assert torch.equal(st, S)
    o2, S2 = sb.fused_recurrent_gla(qd, kd, vd, gd, initial_state=None, output_final_state=False)
    assert S2 is None
    ref_o0, _ = G.gla_recurrent(q.float().numpy(), k.float().numpy(), v.float().numpy(), gate.numpy(), None)
    assert out_close(o2.float().cpu().numpy(), ref_o0)


def test_full_size_config3_properties(sb, dev):
    """BASELINE config 3 (B=64, H=28, fp32 state): properties that need no CPU-sized oracle pass.
    (1) a random sample of (b, h) pairs matches the oracle; (2) linearity of the state update in
    (S, k): step(S1 + S2, k1 + k2) == step(S1, k1) + step(S2, k2) to fp32 rounding."""
    B, H, D = 64, 28, 128
    q, k, v, gate = make(B, H, 1, D, 3)
    g = torch.Generator().manual_seed(9)
    S = torch.randn(B, H, D, D, generator=g) * 0.02
    st = S.clone().to(dev)
    o = sb.my_fused_recurrent_gla(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st,
                                  torch.arange(B, dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    pairs = [(0, 0), (63, 27), (17, 5), (40, 13)]
    for b, h in pairs:
        ref_S = S[b:b + 1, h:h + 1].double().numpy().copy()
        ref_o = G.gla_step(q[b:b + 1, h:h + 1, 0].float().numpy(), k[b:b + 1, h:h + 1, 0].float().numpy(),
                           v[b:b + 1, h:h + 1, 0].float().numpy(), gate[b:b + 1, h:h + 1, 0].numpy(), ref_S)
        assert rel(st[b, h].double().cpu().numpy(), ref_S[0, 0]) <= STATE_RTOL
        assert out_close(o[b, h].float().cpu().numpy(), ref_o[0, 0])
    S2 = torch.randn(B, H, D, D, generator=g) * 0.02
    k2 = torch.randn(B, H, 1, D, generator=g).bfloat16()
    ksum = (k.float() + k2.float())
    a = S.clone().to(dev); b_ = S2.clone().to(dev); c = (S + S2).to(dev)
    qf, vf = q.float().to(dev), v.float().to(dev)
    sb.my_fused_recurrent_gla(qf, k.float().to(dev), vf, gate.to(dev), a, None)
    sb.my_fused_recurrent_gla(qf, k2.float().to(dev), vf, gate.to(dev), b_, None)
    sb.my_fused_recurrent_gla(qf, ksum.to(dev), vf, gate.to(dev), c, None)
    assert ((a + b_ - c).abs().max() / c.abs().max()).item() <= 1e-5


def test_argument_errors(sb, dev):
    q = torch.zeros(2, 4, 1, 128, device=dev, dtype=torch.bfloat16)
    st = torch.zeros(2, 4, 128, 128, device=dev)
    with pytest.raises(ValueError):
        sb.ops.gla_recurrent(q, q[:, :2], q, q, st)
    with pytest.raises(ValueError, match="state must be"):
        sb.ops.gla_recurrent(q, q, q, q, st[:, :2])
    with pytest.raises(NotImplementedError):
        q64 = torch.zeros(2, 4, 1, 64, device=dev, dtype=torch.bfloat16)
        sb.ops.gla_recurrent(q64, q64, q64, q64, torch.zeros(2, 4, 64, 64, device=dev))
    with pytest.raises(RuntimeError, match="no CPU path"):
        sb.ops.gla_recurrent(q.cpu(), q.cpu(), q.cpu(), q.cpu(), st.cpu())


@pytest.mark.parametrize("state_dtype", [torch.float32, torch.bfloat16])
def test_packed_prompts_vs_oracle(sb, dev, state_dtype):
    """Ragged prompts packed token-major [tokens, H, D] (the layout of the vLLM prefill loop,
    vllm_hymeta/model_for_7B/gla_attention.py:179-214): one launch, each prompt starting from its
    slot's state and leaving its final state there; lengths cover 1, below/at/above the 8-step
    register block, and an empty prompt; one slot is -1 (skipped)."""
    H, D = 4, 128
    lens = [1, 7, 8, 9, 0, 37, 16]
    n = len(lens)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    total = int(cu[-1])
    q, k, v, gate = make(1, H, total, D, 77, relu=True)
    q, k, v, gate = (x[0].transpose(0, 1).contiguous() for x in (q, k, v, gate))   # [tokens, H, D]
    g = torch.Generator().manual_seed(3)
    slots = 11
    state = (torch.randn(slots, H, D, D, generator=g) * 0.02).to(state_dtype)
    slot_idx = torch.randperm(slots, generator=g)[:n].to(torch.int32)
    slot_idx[2] = -1
    st = state.clone().to(dev)
    sentinel = 7.0
    out = torch.full((total, H, D), sentinel, dtype=q.dtype, device=dev)
    sb.ops.gla_recurrent_packed(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st, torch.from_numpy(cu).to(dev),
                                slot_idx.to(dev), out=out)
    torch.cuda.synchronize()
    got_o, got_S = out.float().cpu().numpy(), st.double().cpu().numpy()
    tol = STATE_RTOL if state_dtype == torch.float32 else 2 ** -8
    touched = set()
    for i in range(n):
        a, b = int(cu[i]), int(cu[i + 1])
        s = int(slot_idx[i])
        if s < 0:
            assert (got_o[a:b] == sentinel).all()
            continue
        touched.add(s)
        if a == b:
            assert np.array_equal(got_S[s], state[s].double().numpy())
            continue
        hf = lambda x: x[a:b].transpose(0, 1)[None].float().numpy()      # [1, H, T, D]
        ref_o, ref_S = G.gla_recurrent(hf(q), hf(k), hf(v), hf(gate), state[s:s + 1].double().numpy())
        assert rel(got_S[s], ref_S[0]) <= tol, i
        assert out_close(got_o[a:b], ref_o[0].transpose(1, 0, 2)), i
    rest = sorted(set(range(slots)) - touched)
    assert np.array_equal(got_S[rest], state.double().numpy()[rest])


def test_packed_matches_per_prompt_calls_and_wrapper(sb, dev):
    """The packed launch against one call per prompt on the head-first layout: bit-identical where
    both run the same kernel (prompts of 32 tokens or more: the matrix-core block form), within
    tolerance for the 5-token prompt (step-by-step kernel when called alone); `gla_prefill_packed` is
    that launch behind the argument order of the reference's prefill loop."""
    H, D = 28, 128
    lens = [130, 5, 64]
    cu = torch.tensor([0, 130, 135, 199], dtype=torch.int32)
    q, k, v, gate = make(1, H, 199, D, 5)
    q, k, v, gate = (x[0].transpose(0, 1).contiguous().to(dev) for x in (q, k, v, gate))
    cache = torch.zeros(6, H, D, D, device=dev)
    slots = torch.tensor([4, 0, 2, 5], dtype=torch.int32, device=dev)        # one more than prefills
    qsl = torch.tensor([0, 130, 135, 199, 200], dtype=torch.int32, device=dev)
    o = sb.gla.gla_prefill_packed(q, k, v, gate, cache, slots, qsl, num_prefills=3)
    assert o.shape == (199, H, D)
    for i, s in enumerate([4, 0, 2]):
        a, b = int(cu[i]), int(cu[i + 1])
        hf = lambda x: x[a:b].transpose(0, 1).unsqueeze(0)
        o_i, S_i = sb.gla.fused_chunk_gla(hf(q), hf(k), hf(v), hf(gate), initial_state=None, output_final_state=True)
        if b - a >= 32:
            assert torch.equal(S_i[0], cache[s])
            assert torch.equal(o_i[0].transpose(0, 1), o[a:b])
        else:
            assert rel(S_i[0].double().cpu().numpy(), cache[s].double().cpu().numpy()) <= STATE_RTOL
            # two results each within tolerance of the exact one, each rounded to bf16: twice the allowance
            x, y = o_i[0].transpose(0, 1).float().cpu().numpy(), o[a:b].float().cpu().numpy()
            assert bool((np.abs(x - y) <= 2 * OUT_ATOL + 2.0 ** -7 * np.abs(y)).all())
    assert (cache[[1, 3, 5]] == 0).all()


def test_long_prompt_properties(sb, dev):
    """T = 2048 steps: (1) with g = 0 and q = k = e_0 the state's row 0 is the running sum of v
    and o_t = scale * sum_{s<=t} v_s (closed form); (2) splitting the prompt into two calls at a
    step that is not a multiple of the register block reproduces the one-call result bit for bit."""
    B, H, T, D = 2, 3, 2048, 128
    g = torch.Generator().manual_seed(21)
    v = torch.randn(B, H, T, D, generator=g).to(dev)
    e0 = torch.zeros(B, H, T, D, device=dev); e0[..., 0] = 1.0
    zero = torch.zeros(B, H, T, D, device=dev)
    o, S = sb.fused_recurrent_gla(e0, e0, v, zero, scale=1.0, output_final_state=True)
    run = v.double().cumsum(2)
    assert (o.double() - run).abs().max().item() <= 5e-3
    assert (S[:, :, 0].double() - run[:, :, -1]).abs().max().item() <= 5e-3
    assert (S[:, :, 1:] == 0).all()
    q, k, v2, gate = (x.to(dev) for x in make(B, H, T, D, 8, dtype=torch.float32))
    o1, S1 = sb.fused_recurrent_gla(q, k, v2, gate, output_final_state=True)
    cut = 1003
    oa, Sa = sb.fused_recurrent_gla(q[:, :, :cut], k[:, :, :cut], v2[:, :, :cut], gate[:, :, :cut], output_final_state=True)
    ob, Sb = sb.fused_recurrent_gla(q[:, :, cut:], k[:, :, cut:], v2[:, :, cut:], gate[:, :, cut:],
                                    initial_state=Sa, output_final_state=True)
    assert torch.equal(Sb, S1)
    assert torch.equal(torch.cat([oa, ob], 2), o1)


@pytest.mark.parametrize("state_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [32, 33, 47, 100, 256])
def test_block_form_on_matrix_cores_vs_oracle(sb, dev, state_dtype, T):
    """bf16 prompts of 32 steps or more run 16 tokens at a time on the matrix cores: state within
    1e-4 relative (the update's operand is split in two bf16 terms), outputs within 2e-2, against
    the float64 recurrence; the step-by-step fp32 kernel (vector_only) agrees with both."""
    B, H, D = 2, 3, 128
    q, k, v, gate = make(B, H, T, D, 100 + T, relu=True)
    S0 = (torch.randn(5, H, D, D, generator=torch.Generator().manual_seed(T)) * 0.02).to(state_dtype)
    slot_idx = torch.tensor([3, 1], dtype=torch.int32)
    ref_o, ref_S = G.gla_recurrent(q.float().numpy(), k.float().numpy(), v.float().numpy(), gate.numpy(),
                                   S0[slot_idx.long()].double().numpy())
    tol = STATE_RTOL if state_dtype == torch.float32 else 2 ** -8
    for vector_only in (False, True):
        st = S0.clone().to(dev)
        o = sb.ops.gla_recurrent(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st, slot_idx.to(dev), vector_only=vector_only)
        got_S = st.double().cpu().numpy()
        assert rel(got_S[[3, 1]], ref_S) <= tol, vector_only
        assert np.array_equal(got_S[[0, 2, 4]], S0.double().numpy()[[0, 2, 4]])
        assert out_close(o.float().cpu().numpy(), ref_o), vector_only


@pytest.mark.parametrize("strength", [1.5, 3.2])
@pytest.mark.parametrize("gdtype", [torch.float32, torch.bfloat16, torch.float16])
def test_block_form_strong_gates_and_gate_dtypes(sb, dev, gdtype, strength):
    """Gates down to -1.5 per step (exp(-B) reaches e^24 inside a block) and every gate dtype; the
    layout is token-major with a fused q|k|v projection, as the layers produce it. strength 3.2: gates
    uniform in (-3.2, 0), 1.6 per step on average: the kernel applies the decay of the state every second
    block and carries the log-decay of the block in between in the operands' exponents, which then reach
    e^50 to e^75 (the guard clamps at e^80; beyond it results would be wrong, not just imprecise)."""
    B, H, T, D = 1, 2, 70, 128
    g = torch.Generator().manual_seed(5)
    fused = torch.randn(B, T, H, 3 * D, generator=g).bfloat16()
    q, k, v = (fused[..., i * D:(i + 1) * D].transpose(1, 2) for i in range(3))
    gate = (-strength * torch.rand(B, T, H, D, generator=g)).to(gdtype).transpose(1, 2)
    ref_o, ref_S = G.gla_recurrent(q.float().numpy(), k.float().numpy(), v.float().numpy(), gate.float().numpy(), None)
    fd = fused.to(dev)
    qd, kd, vd = (fd[..., i * D:(i + 1) * D].transpose(1, 2) for i in range(3))
    sb.ops.gla_gate_range_hits(reset=True)
    o, S = sb.fused_recurrent_gla(qd, kd, vd, gate.to(dev), output_final_state=True)
    assert rel(S.double().cpu().numpy(), ref_S) <= STATE_RTOL
    assert out_close(o.float().cpu().numpy(), ref_o)
    # the same call with the range check on: same results, nothing counted (inside the block form's range)
    st = torch.zeros(B, H, D, D, device=dev)
    o2 = sb.ops.gla_recurrent(qd, kd, vd, gate.to(dev), st, check_gates=True)
    assert torch.equal(o2, o) and torch.equal(st, S)
    assert sb.ops.gla_gate_range_hits() == 0


def test_gates_beyond_the_block_forms_range_are_counted(sb, dev):
    """32 consecutive log-gates summing below -80 for some key dim put exp(-(cumulative gate)) beyond the exponent
    the block form allows itself: every (prompt, head) workgroup that meets such gates counts itself in the
    device counter that sb_gla_gate_range_hits reads when the call asks for the check (the call itself cannot
    report it: it does not wait for the kernel). Two prompts of a packed launch, one with strong gates in one head only; vector_only has no such
    range and counts nothing."""
    H, D = 2, 128
    lens = [64, 48]
    T = sum(lens)
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(T, H, D, generator=g).bfloat16().to(dev) for _ in range(3))
    gate = -0.5 * torch.rand(T, H, D, generator=g)
    gate[64:112, 1, 5] = -3.0                              # prompt 1, head 1, one key dim: 32 tokens x -3 per pair of blocks
    cu = torch.tensor([0, lens[0], T], dtype=torch.int32, device=dev)
    sb.ops.gla_gate_range_hits(reset=True)
    for vector_only, expect in ((False, 1), (True, 0)):
        state = torch.zeros(2, H, D, D, device=dev)
        sb.ops.gla_recurrent_packed(q, k, v, gate.to(dev), state, cu, max_seq_len=max(lens), vector_only=vector_only,
                                    check_gates=True)
        assert sb.ops.gla_gate_range_hits(reset=True) == expect, vector_only
    # without the flag the kernel is the unchecked build: nothing is counted
    sb.ops.gla_recurrent_packed(q, k, v, gate.to(dev), torch.zeros(2, H, D, D, device=dev), cu, max_seq_len=max(lens))
    assert sb.ops.gla_gate_range_hits() == 0


@pytest.mark.parametrize("gdtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T", [4, 9, 24])
def test_step_by_step_prompt_kernel_every_element_type(sb, dev, dtype, gdtype, T):
    """The many-step vector kernel is compiled once per (q/k/v type, gate type): each of them against the
    oracle, on calls short enough (or of a type) that the matrix-core block form does not take."""
    B, H, D = 2, 3, 128
    q, k, v, gate = make(B, H, T, D, 7 * T, dtype, relu=True)
    gate = gate.to(gdtype)
    S0 = torch.randn(B, H, D, D, generator=torch.Generator().manual_seed(T)) * 0.02
    ref_o, ref_S = G.gla_recurrent(q.float().numpy(), k.float().numpy(), v.float().numpy(), gate.float().numpy(),
                                   S0.double().numpy())
    st = S0.clone().to(dev)
    o = sb.ops.gla_recurrent(q.to(dev), k.to(dev), v.to(dev), gate.to(dev), st)
    assert rel(st.double().cpu().numpy(), ref_S) <= STATE_RTOL
    if dtype == torch.float32:
        assert np.abs(o.double().cpu().numpy() - ref_o).max() <= 1e-4 * max(1.0, np.abs(ref_o).max())
    else:
        assert out_close(o.float().cpu().numpy(), ref_o, dtype)
