"""The hybrid stack's per-token cache work (GLA state layers interleaved with paged sliding-window
layers sharing one block table) stepped next to the oracle: numpy window-cache model, numpy paged
caches, float64 GLA recurrence. Sequences start window-saturated at a long logical context, so
every block_size steps each one evicts a block and recycles its id.
Bit-exact: slot mapping, block tables, view lengths, every byte of every layer's KV tensor.
Within tolerance: attention outputs 2e-2 (bf16); GLA outputs 2e-2 + half an ulp of bf16, states 1e-4 rel."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle import gla as G
from oracle import paged as P

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("ctx", [5, 1000])
def test_hybrid_decode_steps_vs_oracle(sb, dev, ctx):
    B, L, H, HKV, D, bs, wl = 3, 4, 8, 2, 128, 16, 40
    drv = sb.HybridDecodeCache(B, num_layers=L, num_heads=H, num_kv_heads=HKV, head_size=D, block_size=bs,
                               window_left=wl, device=dev, randomize=True, seed=3)
    drv.start(ctx)
    model = P.WindowCacheModel(drv.num_blocks, bs, wl)
    for s in range(B):
        model.add_seq(s)
        model.append_tokens(s, ctx, True)
    kc = [c[0].float().cpu().numpy() for c in drv.kv_caches]
    vc = [c[1].float().cpu().numpy() for c in drv.kv_caches]
    state = drv.gla_state.cpu().numpy().astype(np.float64)
    g = torch.Generator().manual_seed(ctx)
    for step in range(2 * bs + 3):
        meta = drv.step_metadata()
        slots = [model.append_tokens(s, 1, False)[0] for s in range(B)]
        assert meta.slot_mapping.cpu().tolist() == slots
        views = [model.view(s) for s in range(B)]
        lens = [v[1] for v in views]
        assert meta.seq_lens_tensor.cpu().tolist() == lens
        width = max(len(v[0]) for v in views)
        tables = np.zeros((B, width), np.int32)
        for s, v in enumerate(views):
            tables[s, :len(v[0])] = v[0]
        assert np.array_equal(meta.block_tables.cpu().numpy(), tables)
        for li in range(L):
            if li % 2 == 0:
                q, k, v = (torch.randn(B, H, 1, D, generator=g).bfloat16() for _ in range(3))
                gate = torch.nn.functional.logsigmoid(torch.randn(B, H, 1, D, generator=g)) / 16
                o = drv.gla_layer(li, q.to(dev), k.to(dev), v.to(dev), gate.to(dev)).float().cpu().numpy()[:, :, 0]
                ref = G.gla_step(q.float().numpy()[:, :, 0], k.float().numpy()[:, :, 0], v.float().numpy()[:, :, 0],
                                 gate.numpy()[:, :, 0], state[li // 2])
                assert (np.abs(o - ref) <= 2e-2 + np.abs(ref) * 2.0 ** -8).all()
                got_state = drv.gla_state[li // 2].cpu().numpy()
                assert np.abs(got_state - state[li // 2]).max() <= 1e-4 * max(1.0, np.abs(state[li // 2]).max())
            else:
                q = torch.randn(B, H, D, generator=g).bfloat16()
                k = torch.randn(B, HKV, D, generator=g).bfloat16()
                v = torch.randn(B, HKV, D, generator=g).bfloat16()
                out = torch.full((B, H, D), float("nan"), dtype=torch.bfloat16, device=dev)
                drv.swa_layer(li, q.to(dev), k.to(dev), v.to(dev), meta, out)
                j = li // 2
                P.kv_append(k.float().numpy(), v.float().numpy(), kc[j], vc[j], slots)
                ref = A.paged_decode_attention(q.float().numpy(), kc[j], vc[j], tables, lens, D ** -0.5, wl)
                assert np.abs(out.float().cpu().numpy() - ref).max() <= 2e-2
                assert np.array_equal(drv.kv_caches[j][0].float().cpu().numpy(), kc[j])
                assert np.array_equal(drv.kv_caches[j][1].float().cpu().numpy(), vc[j])
    assert drv.manager.free_stack() == model.free


def test_captured_graph_replays_whole_steps(sb, dev):
    """Device-side step advance + all layers captured once in a HIP graph; every replay is one decode
    step on fresh inputs (copied into the static input tensors, with eager work and synchronisation
    between replays) and is checked against the oracle: slots, tables, cache bytes, outputs."""
    B, L, H, HKV, D, bs, wl, ctx = 4, 4, 8, 2, 128, 16, 48, 777
    drv = sb.HybridDecodeCache(B, num_layers=L, num_heads=H, num_kv_heads=HKV, head_size=D, block_size=bs,
                               window_left=wl, device=dev, randomize=True, seed=5)
    drv.start(ctx)
    model = P.WindowCacheModel(drv.num_blocks, bs, wl)
    for s in range(B):
        model.add_seq(s)
        model.append_tokens(s, ctx, True)
    drv.enable_device_advance()
    # static inputs and outputs of the captured step
    gl = [tuple(torch.zeros(B, H, 1, D, dtype=torch.bfloat16, device=dev) for _ in range(3))
          + (torch.zeros(B, H, 1, D, dtype=torch.float32, device=dev),) for _ in range(L // 2)]
    sw = [(torch.zeros(B, H, D, dtype=torch.bfloat16, device=dev), torch.zeros(B, HKV, D, dtype=torch.bfloat16, device=dev),
           torch.zeros(B, HKV, D, dtype=torch.bfloat16, device=dev)) for _ in range(L // 2)]
    g_out = [torch.zeros(B, H, 1, D, dtype=torch.bfloat16, device=dev) for _ in range(L // 2)]
    s_out = [torch.zeros(B, H, D, dtype=torch.bfloat16, device=dev) for _ in range(L // 2)]

    def run_layers(meta):
        for li in range(L):
            if li % 2 == 0:
                drv.gla_layer(li, *gl[li // 2], out=g_out[li // 2])
            else:
                drv.swa_layer(li, *sw[li // 2], meta, s_out[li // 2])

    g = torch.Generator().manual_seed(9)

    def fresh_inputs():
        host = []
        for j in range(L // 2):
            q, k, v = (torch.randn(B, H, 1, D, generator=g).bfloat16() for _ in range(3))
            gate = torch.nn.functional.logsigmoid(torch.randn(B, H, 1, D, generator=g)) / 16
            for dst, src in zip(gl[j], (q, k, v, gate)):
                dst.copy_(src)
            qs = torch.randn(B, H, D, generator=g).bfloat16()
            ks = torch.randn(B, HKV, D, generator=g).bfloat16()
            vs = torch.randn(B, HKV, D, generator=g).bfloat16()
            for dst, src in zip(sw[j], (qs, ks, vs)):
                dst.copy_(src)
            host.append((q, k, v, gate, qs, ks, vs))
        return host

    # the capture's warm-up pass and the capture itself do not execute as checked steps: the warm-up
    # is a real step (oracle follows it), the capture only records
    warm = fresh_inputs()
    graph = drv.capture_step(run_layers)
    torch.cuda.synchronize()
    kc = [c[0].float().cpu().numpy() for c in drv.kv_caches]
    vc = [c[1].float().cpu().numpy() for c in drv.kv_caches]
    state = drv.gla_state.cpu().numpy().astype(np.float64)
    for s in range(B):
        model.append_tokens(s, 1, False)        # the warm-up step (its cache writes are in kc/vc already)
    del warm
    for step in range(2 * bs + 2):
        host = fresh_inputs()
        graph.replay()
        torch.cuda.synchronize()
        slots = [model.append_tokens(s, 1, False)[0] for s in range(B)]
        assert drv.device_state.slot_mapping.cpu().tolist() == slots, f"replay {step}"
        views = [model.view(s) for s in range(B)]
        lens = [v[1] for v in views]
        assert drv.device_state.seq_lens.cpu().tolist() == lens
        tables = np.zeros((B, drv.device_state.table_width), np.int32)
        for s, v in enumerate(views):
            tables[s, :len(v[0])] = v[0]
        assert np.array_equal(drv.device_state.block_tables.cpu().numpy(), tables)
        for j in range(L // 2):
            q, k, v, gate, qs, ks, vs = host[j]
            ref = G.gla_step(q.float().numpy()[:, :, 0], k.float().numpy()[:, :, 0], v.float().numpy()[:, :, 0],
                             gate.numpy()[:, :, 0], state[j])
            o = g_out[j].float().cpu().numpy()[:, :, 0]
            assert (np.abs(o - ref) <= 2e-2 + np.abs(ref) * 2.0 ** -8).all()
            P.kv_append(ks.float().numpy(), vs.float().numpy(), kc[j], vc[j], slots)
            ref = A.paged_decode_attention(qs.float().numpy(), kc[j], vc[j], tables, lens, D ** -0.5, wl)
            assert np.abs(s_out[j].float().cpu().numpy() - ref).max() <= 2e-2, f"replay {step} layer {2 * j + 1}"
            assert np.array_equal(drv.kv_caches[j][0].float().cpu().numpy(), kc[j])
    drv.device_state.download()
    assert drv.manager.free_stack() == model.free


def test_shared_gla_states_give_the_same_outputs(sb, dev):
    """One GLA state per kv head: the driver takes k, v and the gate before the model's repeat_kv
    (vllm_hymeta/model_for_7B/gla_attention.py:264-267) and must give, bit for bit, what the 28-state
    driver gives on the repeated tensors; bytes_per_step counts the smaller state traffic."""
    B, L, H, HKV, D = 5, 4, 28, 4, 128
    kw = dict(num_layers=L, num_heads=H, num_kv_heads=HKV, head_size=D, window_left=40, device=dev)
    shared = sb.HybridDecodeCache(B, randomize=True, seed=9, gla_shared_states=True, **kw)
    full = sb.HybridDecodeCache(B, **kw)
    assert shared.gla_state.shape == (L // 2, B, HKV, D, D) and full.gla_state.shape == (L // 2, B, H, D, D)
    full.gla_state.copy_(shared.gla_state.repeat_interleave(H // HKV, dim=2))
    g = torch.Generator().manual_seed(0)
    for step in range(4):
        for li in (0, 2):
            q = torch.randn(B, H, 1, D, generator=g).bfloat16().to(dev)
            k, v = (torch.randn(B, HKV, 1, D, generator=g).bfloat16().to(dev) for _ in range(2))
            gate = (torch.nn.functional.logsigmoid(torch.randn(B, HKV, 1, D, generator=g)) / 16).to(dev)
            o = shared.gla_layer(li, q, k, v, gate).clone()
            r = H // HKV
            o_full = full.gla_layer(li, q, k.repeat_interleave(r, 1), v.repeat_interleave(r, 1),
                                    gate.repeat_interleave(r, 1))
            assert torch.equal(o, o_full), (step, li)
    assert torch.equal(shared.gla_state, full.gla_state[:, :, ::H // HKV])
    shared.start(100)
    full.start(100)
    e = 2
    per_layer_saving = B * (H - HKV) * (2 * D * D * 4 + 2 * D * e + D * 4)
    assert full.bytes_per_step() - shared.bytes_per_step() == (L // 2) * per_layer_saving
