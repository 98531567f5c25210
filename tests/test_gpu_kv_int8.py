"""Per-row INT8 K/V: codes and scales bit-exact against the oracle (integer/byte work), decode
attention over the INT8 cache within 2e-2 of the oracle's attention over the dequantised rows."""
import numpy as np
import pytest
import torch

from oracle import attention as A
from oracle import quant as Q

pytestmark = pytest.mark.gpu

D = 128


def rows(T, H, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, D, generator=g) * (10 ** torch.empty(T, H, 1).uniform_(-3, 2, generator=g))
    x[0, 0] = 0                                  # scale clamps to 1e-5
    if T > 2:
        x[1, 0, :3] = torch.tensor([3e6, -3e6, 1.5e4])   # scale clamps to 1e4, codes saturate
        x[2, 0, :4] = torch.tensor([127.0, 63.5, 62.5, -62.5]); x[2, 0, 4:] = 0   # ties
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H", [4, 2, 7])
def test_append_int8_bit_exact(sb, dev, dtype, H):
    nb, bs, T = 9, 16, 40
    k, v = rows(T, H, 1, dtype), rows(T, H, 2, dtype)
    g = torch.Generator().manual_seed(3)
    slots = torch.randperm(nb * bs, generator=g)[:T]
    slots[5] = -1
    kv, sc = sb.ops.alloc_int8_kv_cache(nb, bs, H, D, dev)
    kv.fill_(3); sc.fill_(-1.0)
    ref_kv = kv.cpu().numpy().copy(); ref_sc = sc.cpu().numpy().copy()
    Q.kv_append_int8(k.float().numpy(), v.float().numpy(), ref_kv[0], ref_kv[1], ref_sc[0], ref_sc[1], slots.tolist())
    # token-major views of a fused projection, as the layers produce them
    fused = torch.cat([k, v], 1).to(dev)
    sb.ops.kv_append_int8(fused[:, :H], fused[:, H:], kv[0], kv[1], sc[0], sc[1], slots.to(dev))
    assert np.array_equal(kv.cpu().numpy(), ref_kv)
    assert np.array_equal(sc.cpu().numpy(), ref_sc)


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16"), (torch.float16, "f16"), (torch.float32, "f32")])
def test_quantize_sym_bit_exact(sb, dev, dtype, name):
    x = rows(33, 4, 7, dtype)
    ref = Q.quantize_sym(x.float().numpy(), name)
    xd = x.to(dev)
    y = sb.ops.quantize_sym(xd)
    assert np.array_equal(y.float().cpu().numpy(), ref)
    sb.ops.quantize_sym(xd, out=xd)              # in place
    assert torch.equal(xd, y)


def int8_problem(sb, dev, lens, bs, Hkv, dtype, seed):
    """Paged INT8 cache holding lens[b] keys per sequence, filled through kv_append_int8; returns the
    device tensors and the oracle's float view of what attention should see (dequantised rows)."""
    g = torch.Generator().manual_seed(seed)
    need = [(n + bs - 1) // bs for n in lens]
    nb = sum(need) + 3
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(len(lens), max(max(need), 1), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
    T = sum(lens)
    k = (torch.randn(T, Hkv, D, generator=g) * (0.5 + torch.rand(T, Hkv, 1, generator=g))).to(dtype)
    v = (torch.randn(T, Hkv, D, generator=g) * (1 + torch.rand(T, Hkv, 1, generator=g))).to(dtype)
    slots = torch.cat([torch.tensor([int(tables[b, i // bs]) * bs + i % bs for i in range(n)], dtype=torch.int64)
                       for b, n in enumerate(lens)]) if T else torch.zeros(0, dtype=torch.int64)
    kv, sc = sb.ops.alloc_int8_kv_cache(nb, bs, Hkv, D, dev)
    sc.fill_(float("nan"))                      # rows never written must not leak into any result
    sb.ops.kv_append_int8(k.to(dev), v.to(dev), kv[0], kv[1], sc[0], sc[1], slots.to(dev))
    name = {torch.bfloat16: "bf16", torch.float16: "f16"}[dtype]
    views = []
    for rounding in (name, "f32"):      # as the reference rounds them (to the tensor's dtype) / code * scale exactly
        kd = Q.quantize_sym(k.float().numpy(), rounding); vd = Q.quantize_sym(v.float().numpy(), rounding)
        kc = np.zeros((nb, bs, Hkv, D)); vc = np.zeros((nb, bs, Hkv, D))
        for t, s in enumerate(slots.tolist()):
            kc[s // bs, s % bs] = kd[t]; vc[s // bs, s % bs] = vd[t]
        views.append((kc, vc))
    return kv, sc, tables, views


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hq,Hkv", [(28, 4), (8, 8), (16, 2)])
@pytest.mark.parametrize("wl,n_split", [(64, 1), (100, 3), (-1, 2), (0, 1)])
def test_decode_over_int8_cache_vs_oracle(sb, dev, dtype, Hq, Hkv, wl, n_split):
    bs = 16
    lens = [1, 17, 64, 65, 300, 0, 129]
    kv, sc, tables, views = int8_problem(sb, dev, lens, bs, Hkv, dtype, Hq + wl)
    g = torch.Generator().manual_seed(1)
    q = torch.randn(len(lens), Hq, D, generator=g).to(dtype)
    scale = D ** -0.5
    (ref, ref_lse), (exact, exact_lse) = (A.paged_decode_attention(q.float().numpy(), kc, vc, tables.numpy(), lens, scale,
                                                                   wl, return_lse=True) for kc, vc in views)
    out, lse = sb.ops.swa_decode_attention(q.to(dev), kv[0], kv[1], torch.tensor(lens, dtype=torch.int32, device=dev),
                                           block_table=tables.to(dev), window_left=wl, scale=scale, n_split=n_split,
                                           k_scale=sc[0], v_scale=sc[1], return_lse=True)
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any()
    live = [b for b, n in enumerate(lens) if n > 0]
    # 2e-2 max-abs on the fp32 result, plus the half ulp that storing it in the 16-bit type adds
    # (|o| reaches 5 here: V rows are scaled by 1..2)
    ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    assert (np.abs(got[live] - ref[live]) <= 2e-2 + ulp * np.abs(ref[live])).all()
    # The reference rounds code * scale to the tensor's dtype before attending; the kernel applies the
    # scales in fp32 to scores and probabilities. Against the unrounded rows it is therefore tighter.
    assert np.abs(lse.cpu().numpy()[live] - ref_lse[live]).max() <= 1e-2
    assert np.abs(lse.cpu().numpy()[live] - exact_lse[live]).max() <= 2e-3
    assert (np.abs(got[live] - exact[live]) <= 2e-2 + ulp * np.abs(exact[live])).all()
    assert (got[5] == 0).all()


def test_int8_cache_argument_errors(sb, dev):
    kv, sc = sb.ops.alloc_int8_kv_cache(4, 16, 4, D, dev)
    q = torch.zeros(2, 28, D, dtype=torch.bfloat16, device=dev)
    sl = torch.ones(2, dtype=torch.int32, device=dev)
    bt = torch.zeros(2, 2, dtype=torch.int32, device=dev)
    with pytest.raises(ValueError):
        sb.ops.swa_decode_attention(q, kv[0], kv[1], sl, block_table=bt, k_scale=sc[0])
    with pytest.raises(NotImplementedError):
        sb.ops.swa_decode_attention(q.float(), kv[0], kv[1], sl, block_table=bt, k_scale=sc[0], v_scale=sc[1])
    with pytest.raises(NotImplementedError):
        sb.ops.swa_decode_attention(q, kv[0], kv[1], sl, block_table=bt, k_scale=sc[0], v_scale=sc[1],
                                    new_key=q[:, :4], new_value=q[:, :4], new_slot_mapping=torch.zeros(2, dtype=torch.int64, device=dev))
    with pytest.raises(ValueError):
        sb.ops.kv_append_int8(q[:, :4], q[:, :4], kv[0], kv[1], sc[0][:, :2], sc[1], torch.zeros(2, dtype=torch.int64, device=dev))


def test_hybrid_decode_driver_with_int8_kv(sb, dev):
    """The decode driver with kv_quant="int8": every step appends quantised rows and attends over the
    INT8 cache; host-stepped and device-advanced runs leave identical caches and outputs, and the
    outputs match the oracle's attention over the dequantised history of one sequence."""
    B, wl, bs = 3, 40, 16
    runs = []
    for device_advance in (False, True):
        c = sb.HybridDecodeCache(B, num_layers=2, window_left=wl, block_size=bs, device=dev, kv_quant="int8")
        c.start(0)
        g = torch.Generator().manual_seed(9)
        hist_k, hist_v, outs = [], [], []
        meta = c.enable_device_advance() if device_advance else None
        for step in range(3 * bs):
            q = torch.randn(B, 28, D, generator=g).bfloat16()
            k = torch.randn(B, 4, D, generator=g).bfloat16()
            v = torch.randn(B, 4, D, generator=g).bfloat16()
            if device_advance:
                c.advance_device()
            else:
                meta = c.step_metadata()
            out = torch.empty(B, 28, D, dtype=torch.bfloat16, device=dev)
            c.swa_layer(1, q.to(dev), k.to(dev), v.to(dev), meta, out)
            hist_k.append(k[0]); hist_v.append(v[0]); outs.append(out.cpu())
            if step in (0, wl + 3, 3 * bs - 1):
                kd = Q.quantize_sym(torch.stack(hist_k).float().numpy(), "bf16")
                vd = Q.quantize_sym(torch.stack(hist_v).float().numpy(), "bf16")
                ref = A.varlen_window_attention(q[0:1].float().numpy(), kd, vd, [0, 1], [0, len(kd)], D ** -0.5, wl)
                assert np.abs(out[0:1].float().cpu().numpy() - ref).max() <= 2e-2, step
        runs.append((torch.stack(outs), c.kv_caches[0].cpu(), c.kv_scales[0].cpu()))
    assert torch.equal(runs[0][0], runs[1][0])
    assert torch.equal(runs[0][1], runs[1][1]) and torch.equal(runs[0][2], runs[1][2])


def test_backend_engine_with_int8_cache(sb, dev):
    """Prompt step, chunked second prompt + decodes, decode steps with eviction, through
    MetaAttentionImpl.forward on Int8KVCache layers: codes and scales bit-exact against the oracle's
    quantised append at the oracle's slots; outputs within 2e-2 of attention over the rows as
    quantize_sym returns them (what the W8ASpike layer attends to)."""
    from oracle import paged as P
    HQ, HKV, bs, wl, nb = 28, 4, 16, 40, 48
    runner = sb.runner.SwaCacheRunner(1, nb, bs, wl, HKV, D, torch.bfloat16, dev, max_seqs=3, max_chunk_tokens=128,
                                      kv_quant="int8")
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, wl + 1, "auto")
    model = P.WindowCacheModel(nb, bs, wl)
    kc = np.zeros((nb, bs, HKV, D), np.int8); vc = np.zeros_like(kc)
    ks = np.zeros((nb, HKV, bs), np.float32); vs = np.zeros_like(ks)
    hist = {}
    g = torch.Generator().manual_seed(11)

    def step(prompts, decodes, chunked=False):
        T = sum(n for _, n in prompts) + len(decodes)
        q = torch.randn(T, HQ, D, generator=g).bfloat16()
        k = torch.randn(T, HKV, D, generator=g).bfloat16()
        v = torch.randn(T, HKV, D, generator=g).bfloat16()
        meta = runner.build_step(prompts, decodes, chunked_prefill=chunked)
        slots = []
        for sid, n in prompts:
            slots += model.append_tokens(sid, n, True, store_all=chunked)
        for sid in decodes:
            slots += model.append_tokens(sid, 1, False)
        assert meta.slot_mapping.cpu().tolist() == slots
        Q.kv_append_int8(k.float().numpy(), v.float().numpy(), kc, vc, ks, vs, slots)
        out = torch.full((T, HQ, D), float("nan"), dtype=torch.bfloat16, device=dev)
        impl.forward(None, q.to(dev), k.to(dev), v.to(dev), None, None, None, runner.kv_caches[0], meta, output=out)
        cache = runner.kv_caches[0]
        assert np.array_equal(cache.codes[0].cpu().numpy(), kc) and np.array_equal(cache.codes[1].cpu().numpy(), vc)
        written = ks != 0
        assert np.array_equal(cache.scales[0].cpu().numpy()[written], ks[written])
        assert np.array_equal(cache.scales[1].cpu().numpy()[written], vs[written])
        got = out.float().cpu().numpy()
        t = 0
        for sid, n in list(prompts) + [(s, 1) for s in decodes]:
            hk, hv = hist.get(sid, (np.zeros((0, HKV, D), np.float32), np.zeros((0, HKV, D), np.float32)))
            hk = np.concatenate([hk, Q.quantize_sym(k[t:t + n].float().numpy(), "bf16")])
            hv = np.concatenate([hv, Q.quantize_sym(v[t:t + n].float().numpy(), "bf16")])
            hist[sid] = (hk, hv)
            ref = A.varlen_window_attention(q[t:t + n].float().numpy(), hk, hv, [0, n], [0, len(hk)], D ** -0.5, wl)
            assert np.abs(got[t:t + n] - ref).max() <= 2e-2 + 2.0 ** -8 * np.abs(ref).max(), (sid, n)
            t += n

    for sid in (0, 1, 2):
        runner.add_seq(sid); model.add_seq(sid)
    step([(0, 25), (1, 90)], [])                       # plain prompts: attention over the quantised in-flight rows
    step([(2, 50)], [0, 1], chunked=True)              # chunked prompt reads the INT8 paged cache + two decodes
    for _ in range(bs + 3):
        step([], [0, 1, 2])
    # copy-on-write block copy moves codes and scales together
    src = int(runner.kv_caches[0].scales[0].abs().sum((1, 2)).argmax())
    dst = model.free[-1] if hasattr(model, "free") and model.free else (src + 1) % nb
    before = runner.kv_caches[0].codes[:, src].clone(), runner.kv_caches[0].scales[:, src].clone()
    sb.MetaAttentionBackend.copy_blocks(runner.kv_caches, torch.tensor([[src, dst]], dtype=torch.int64, device=dev))
    assert torch.equal(runner.kv_caches[0].codes[:, dst], before[0]) and torch.equal(runner.kv_caches[0].scales[:, dst], before[1])


# ---------------------------------------------------------------- fp8 (e4m3fn) cache
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("scales", [(1.0, 1.0), (0.5, 0.03125)])
def test_append_fp8_and_round_bit_exact(sb, dev, dtype, scales):
    nb, bs, T, H = 6, 16, 30, 4
    g = torch.Generator().manual_seed(21)
    k = (torch.randn(T, H, D, generator=g) * 10 ** torch.empty(T, H, 1).uniform_(-3, 2.5, generator=g)).to(dtype)
    v = (torch.randn(T, H, D, generator=g) * 3).to(dtype)
    k[0, 0, :6] = torch.tensor([448.0, 464.0, 1000.0, -3000.0, 2.0 ** -9, 1.5 * 2.0 ** -9]).to(dtype)   # saturation, subnormals, a tie
    slots = torch.randperm(nb * bs, generator=g)[:T]
    slots[3] = -1
    kc = torch.full((2, nb, bs, H, D), 0x11, dtype=torch.uint8, device=dev)
    ref = kc.cpu().numpy().copy()
    codes_k = Q.fp8_codes(k.float().numpy(), scales[0]); codes_v = Q.fp8_codes(v.float().numpy(), scales[1])
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            ref[0, s // bs, s % bs] = codes_k[t]; ref[1, s // bs, s % bs] = codes_v[t]
    cache = kc.view(torch.float8_e4m3fn)
    sb.ops.kv_append_fp8(k.to(dev), v.to(dev), cache[0], cache[1], slots.to(dev), *scales)
    assert np.array_equal(kc.cpu().numpy(), ref)
    name = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[dtype]
    got = sb.ops.fp8_round(k.to(dev), scales[0]).float().cpu().numpy()
    assert np.array_equal(got, Q.fp8_round(k.float().numpy(), scales[0], name))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hq,Hkv", [(28, 4), (16, 2)])
@pytest.mark.parametrize("wl,n_split,scales", [(64, 1, (1.0, 1.0)), (100, 3, (0.25, 0.5)), (-1, 2, (1.0, 1.0))])
def test_decode_over_fp8_cache_vs_oracle(sb, dev, dtype, Hq, Hkv, wl, n_split, scales):
    bs = 16
    lens = [1, 17, 64, 65, 300, 0, 129]
    g = torch.Generator().manual_seed(Hq + wl)
    need = [(n + bs - 1) // bs for n in lens]
    nb = sum(need) + 3
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(len(lens), max(need), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
    T = sum(lens)
    k = torch.randn(T, Hkv, D, generator=g).to(dtype)
    v = (torch.randn(T, Hkv, D, generator=g) * 1.5).to(dtype)
    slots = torch.cat([torch.tensor([int(tables[b, i // bs]) * bs + i % bs for i in range(n)], dtype=torch.int64)
                       for b, n in enumerate(lens)])
    raw = torch.full((2, nb, bs, Hkv, D), 0x7F, dtype=torch.uint8, device=dev)      # every unwritten byte is a NaN code
    cache = raw.view(torch.float8_e4m3fn)
    sb.ops.kv_append_fp8(k.to(dev), v.to(dev), cache[0], cache[1], slots.to(dev), *scales)
    kc = np.zeros((nb, bs, Hkv, D)); vc = np.zeros((nb, bs, Hkv, D))
    kd = Q.fp8_values(Q.fp8_codes(k.float().numpy(), scales[0]), scales[0])
    vd = Q.fp8_values(Q.fp8_codes(v.float().numpy(), scales[1]), scales[1])
    for t, s in enumerate(slots.tolist()):
        kc[s // bs, s % bs] = kd[t]; vc[s // bs, s % bs] = vd[t]
    q = torch.randn(len(lens), Hq, D, generator=g).to(dtype)
    scale = D ** -0.5
    ref, ref_lse = A.paged_decode_attention(q.float().numpy(), kc, vc, tables.numpy(), lens, scale, wl, return_lse=True)
    out, lse = sb.ops.swa_decode_attention(q.to(dev), cache[0], cache[1], torch.tensor(lens, dtype=torch.int32, device=dev),
                                           block_table=tables.to(dev), window_left=wl, scale=scale, n_split=n_split,
                                           fp8_scales=scales, return_lse=True)
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any()
    live = [b for b, n in enumerate(lens) if n > 0]
    ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    assert (np.abs(got[live] - ref[live]) <= 2e-2 + ulp * np.abs(ref[live])).all()
    assert np.abs(lse.cpu().numpy()[live] - ref_lse[live]).max() <= 2e-3
    assert (got[5] == 0).all()


def test_backend_engine_with_fp8_cache(sb, dev):
    """kv_cache_dtype="fp8" through MetaAttentionImpl.forward with layer scales: codes bit-exact against
    the oracle's fp8 append at the oracle's slots; outputs within 2e-2 of attention computed from the
    query, keys and values after their fp8 round trips (the reference quantises all three)."""
    from oracle import paged as P
    HQ, HKV, bs, wl, nb = 28, 4, 16, 40, 48
    runner = sb.runner.SwaCacheRunner(1, nb, bs, wl, HKV, D, torch.uint8, dev, max_seqs=3, max_chunk_tokens=128)
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, wl + 1, "fp8")

    class Layer:
        _k_scale_float, _v_scale_float, _q_scale_float = 0.5, 0.25, 0.125

    ks, vs, qs = Layer._k_scale_float, Layer._v_scale_float, Layer._q_scale_float
    model = P.WindowCacheModel(nb, bs, wl)
    kc = np.zeros((nb, bs, HKV, D), np.uint8); vc = np.zeros_like(kc)
    hist = {}
    g = torch.Generator().manual_seed(12)

    def step(prompts, decodes, chunked=False):
        T = sum(n for _, n in prompts) + len(decodes)
        q = torch.randn(T, HQ, D, generator=g).bfloat16()
        k = torch.randn(T, HKV, D, generator=g).bfloat16()
        v = torch.randn(T, HKV, D, generator=g).bfloat16()
        meta = runner.build_step(prompts, decodes, chunked_prefill=chunked)
        slots = []
        for sid, n in prompts:
            slots += model.append_tokens(sid, n, True, store_all=chunked)
        for sid in decodes:
            slots += model.append_tokens(sid, 1, False)
        ck, cv = Q.fp8_codes(k.float().numpy(), ks), Q.fp8_codes(v.float().numpy(), vs)
        for t, s in enumerate(slots):
            if s >= 0:
                kc[s // bs, s % bs] = ck[t]; vc[s // bs, s % bs] = cv[t]
        out = torch.full((T, HQ, D), float("nan"), dtype=torch.bfloat16, device=dev)
        impl.forward(Layer(), q.to(dev), k.to(dev), v.to(dev), None, None, None, runner.kv_caches[0], meta, output=out)
        assert np.array_equal(runner.kv_caches[0][0].cpu().numpy(), kc) and np.array_equal(runner.kv_caches[0][1].cpu().numpy(), vc)
        got = out.float().cpu().numpy()
        qr = Q.fp8_round(q.float().numpy(), qs, "bf16")
        t = 0
        for sid, n in list(prompts) + [(s, 1) for s in decodes]:
            hk, hv = hist.get(sid, (np.zeros((0, HKV, D), np.float32), np.zeros((0, HKV, D), np.float32)))
            hk = np.concatenate([hk, Q.fp8_round(k[t:t + n].float().numpy(), ks, "f32")])
            hv = np.concatenate([hv, Q.fp8_round(v[t:t + n].float().numpy(), vs, "f32")])
            hist[sid] = (hk, hv)
            ref = A.varlen_window_attention(qr[t:t + n], hk, hv, [0, n], [0, len(hk)], D ** -0.5, wl)
            assert np.abs(got[t:t + n] - ref).max() <= 2e-2 + 2.0 ** -8 * np.abs(ref).max(), (sid, n)
            t += n

    for sid in (0, 1, 2):
        runner.add_seq(sid); model.add_seq(sid)
    step([(0, 25), (1, 90)], [])
    step([(2, 50)], [0, 1], chunked=True)
    for _ in range(bs + 3):
        step([], [0, 1, 2])
    with pytest.raises(NotImplementedError):
        sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, wl + 1, "fp8_e5m2")


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("Hq,Hkv", [(28, 4), (8, 8)])
def test_prefill_kernel_over_byte_code_caches(sb, dev, kind, Hq, Hkv):
    """Chunked prefill reading an INT8 / fp8 paged cache with the many-query kernel: rows are
    dequantised into the kernel's LDS stage; compared with the oracle's attention over the rows as the
    reference's quantise-dequantise leaves them (code * scale rounded to bf16)."""
    bs, wl = 16, 70
    qlens, klens = [40, 5, 130], [100, 5, 230]           # second and third chunks of prompts, one whole short prompt
    g = torch.Generator().manual_seed(31)
    need = [(n + bs - 1) // bs for n in klens]
    nb = sum(need) + 2
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(len(klens), max(need), dtype=torch.int32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]; p += n
    Tk, Tq = sum(klens), sum(qlens)
    k = (torch.randn(Tk, Hkv, D, generator=g) * (0.5 + torch.rand(Tk, Hkv, 1, generator=g))).bfloat16()
    v = (torch.randn(Tk, Hkv, D, generator=g) * (1 + torch.rand(Tk, Hkv, 1, generator=g))).bfloat16()
    q = torch.randn(Tq, Hq, D, generator=g).bfloat16()
    slots = torch.cat([torch.tensor([int(tables[b, i // bs]) * bs + i % bs for i in range(n)], dtype=torch.int64)
                       for b, n in enumerate(klens)])
    if kind == "int8":
        kv, sc = sb.ops.alloc_int8_kv_cache(nb, bs, Hkv, D, dev)
        sc.fill_(float("nan"))
        sb.ops.kv_append_int8(k.to(dev), v.to(dev), kv[0], kv[1], sc[0], sc[1], slots.to(dev))
        kw = dict(k_scale=sc[0], v_scale=sc[1])
        kd, vd = Q.quantize_sym(k.float().numpy(), "bf16"), Q.quantize_sym(v.float().numpy(), "bf16")
    else:
        raw = torch.full((2, nb, bs, Hkv, D), 0x7F, dtype=torch.uint8, device=dev)
        kv = raw.view(torch.float8_e4m3fn)
        sb.ops.kv_append_fp8(k.to(dev), v.to(dev), kv[0], kv[1], slots.to(dev), 0.5, 0.25)
        kw = dict(fp8_scales=(0.5, 0.25))
        kd, vd = Q.fp8_round(k.float().numpy(), 0.5, "bf16"), Q.fp8_round(v.float().numpy(), 0.25, "bf16")
    out, lse = sb.ops.swa_prefill_attention(q.to(dev), kv[0], kv[1], query_lens=qlens, seq_lens_k=klens,
                                            block_table=tables.to(dev), window_left=wl, return_lse=True, **kw)
    cu_q = np.concatenate([[0], np.cumsum(qlens)]); cu_k = np.concatenate([[0], np.cumsum(klens)])
    ref = A.varlen_window_attention(q.float().numpy(), kd, vd, cu_q, cu_k, D ** -0.5, wl)
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any() and not torch.isnan(lse).any()
    assert (np.abs(got - ref) <= 2e-2 + 2.0 ** -8 * np.abs(ref)).all()
