"""Benchmark of the decode-time cache hot path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input at BASELINE config 2
(paged SWA decode at the 7B layer shape): KV append of one new token per sequence through
slot_mapping, then window-bounded paged decode attention (split kernel + merge kernel); for a pure
decode batch the split kernel does the append itself (one launch less), as the backend's forward does.
  B=64, 28 q / 4 kv heads, head_dim 128, block_size 16, window_left 4096, bf16,
  context lengths ~ U[1024, 32768] (seed 0), seeded block permutation, only in-window blocks
  resident, K/V ~ N(0,1).
`value` is algorithmic bytes of a step / wall time of a step, inputs resident in HBM.
Between steps the bench rotates over several copies of the KV cache whose total size exceeds
the 256 MB on-die cache, so every step reads its K/V from HBM.

Prints ONE JSON line (rank 0 is the only rank: this build is single-GPU).
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the matrix-core split kernel at the default workload come from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs (counters cannot be read from inside this script). The profile summary records
# them together with a hash of the kernel sources it was taken with; the figure is attached to the bench line
# only while the sources still hash to that value.
PROFILE_FILE = os.path.join(ROOT, "profiles", "swa_decode_stream_config2.md")
KERNEL_SOURCES = ("swa_decode_stream.hip", "swa_decode.hip", "swa_decode_params.h", "mfma_util.h", "common.h")


def kernel_sources_hash():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "spikingbrain-7b_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def recorded_traffic():
    """(bytes per launch or None, where the figure comes from)."""
    import re
    try:
        text = open(PROFILE_FILE).read()
    except OSError:
        return None, "no profile summary"
    m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)\s*;\s*kernel_sources_sha256_16\s*=\s*([0-9a-f]{16})", text)
    if not m:
        return None, "profile summary holds no traffic record"
    if m.group(2) != kernel_sources_hash():
        return None, "profiles/swa_decode_stream_config2.md was recorded with older kernel sources"
    return int(m.group(1)), "rocprofv3 FETCH_SIZE + WRITE_SIZE recorded in profiles/swa_decode_stream_config2.md (same kernel sources)"


HQ, HKV, D, BS, WL = 28, 4, 128, 16, 4096
E = 2  # bf16


def build_config2(dev, B=64, seed=0, copies=3):
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(1024, 32769, (B,), generator=g)          # tokens already cached
    pos = ctx                                                    # position of the new token
    lo_blk = torch.clamp((pos - WL) // BS, min=0)
    hi_blk = pos // BS
    nblk = hi_blk - lo_blk + 1
    nb = int(int(nblk.sum()) * 1.1) + 1
    perm = torch.randperm(nb, generator=g)
    tables = torch.zeros(B, int(nblk.max()), dtype=torch.int32)
    p = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[p:p + int(nblk[b])]
        p += int(nblk[b])
    seqlens = (pos + 1 - lo_blk * BS).to(torch.int32)            # view-relative length incl. the new token
    k_idx = pos - lo_blk * BS                                    # view-relative index of the new token
    slots = tables[torch.arange(B), (k_idx // BS).long()].to(torch.int64) * BS + k_idx % BS
    n_keys = torch.minimum(pos + 1, torch.tensor(WL + 1))        # keys each query attends to
    kv = [torch.randn(2, nb, BS, HKV, D, device=dev, dtype=torch.bfloat16) for _ in range(copies)]
    prob = dict(
        B=B, nb=nb, kv=kv, tables=tables.to(dev), seqlens=seqlens.to(dev), slots=slots.to(dev),
        q=torch.randn(B, HQ, D, device=dev, dtype=torch.bfloat16),
        k=torch.randn(B, HKV, D, device=dev, dtype=torch.bfloat16),
        v=torch.randn(B, HKV, D, device=dev, dtype=torch.bfloat16),
        out=torch.empty(B, HQ, D, device=dev, dtype=torch.bfloat16),
        n_keys=n_keys, max_seq_len=int(seqlens.max()), resident_blocks=int(nblk.sum()))
    # algorithmic bytes of one layer-step (formula of the measurement plan):
    kv_read = int(n_keys.sum()) * HKV * D * 2 * E               # K and V rows inside the window
    qo = 2 * B * HQ * D * E                                      # q read, o write
    new_kv = 2 * B * HKV * D * E * 2                             # new k,v read + written to the cache
    tables_b = int(nblk.sum()) * 4 + B * (8 + 4)                 # block ids, slot, seq_len
    prob["bytes_step"] = kv_read + qo + new_kv + tables_b
    prob["bytes_split_kernel"] = kv_read + qo + int(nblk.sum()) * 4 + B * 4
    return prob


def cpu_baseline(seconds_budget=12.0, sample_B=8):
    """The reference's PyTorch CPU path (oracle/cpu_path.py, a port) on a bounded sample of the
    same workload: sample_B sequences, window-saturated dense fp32 caches [B, 4, 4097, 128], one
    decode token: roll + slice-assign update, repeat_kv, SDPA with the sliding-causal mask."""
    from oracle import cpu_path

    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    W = WL + 1
    k_state = torch.randn(sample_B, HKV, W, D, generator=g)
    v_state = torch.randn(sample_B, HKV, W, D, generator=g)
    q = torch.randn(sample_B, HQ, 1, D, generator=g)
    k_new = torch.randn(sample_B, HKV, 1, D, generator=g)
    v_new = torch.randn(sample_B, HKV, 1, D, generator=g)
    times = []
    t_end = time.perf_counter() + seconds_budget
    it = 0
    while it < 3 or (time.perf_counter() < t_end and it < 200):
        t0 = time.perf_counter()
        k_state, v_state = cpu_path.dense_window_update(k_state, v_state, k_new, v_new, W)
        cpu_path.sdpa_window_attention(q, k_state, v_state, W)
        dt = time.perf_counter() - t0
        if it >= 2:
            times.append(dt)
        it += 1
    med = statistics.median(times)
    # same algorithmic-byte formula as the GPU line (bf16 element size) so the unit is comparable
    bytes_sample = sample_B * (W * HKV * D * 2 * E + 2 * HQ * D * E + 2 * HKV * D * E * 2 + (W // BS + 1) * 4 + 12)
    return dict(value=bytes_sample / med / 1e9, unit="GB/s", cores=threads, kind="port",
                sample=f"{sample_B} of 64 sequences, window-saturated (4097 keys), fp32 dense cache, "
                       f"cache.py roll update + repeat_kv + SDPA, median of {len(times)} steps, "
                       f"{med * 1e3:.1f} ms/step")


MFMA_BF16_PEAK_TFLOPS = 2500.0


def bench_prefill(sb, dev, S=16, L=8192, iters=5):
    """BASELINE config 4 through the backend: 16 prompts x 8192 new tokens, window_left 4096, one layer.
    Times MetaAttentionImpl.forward (bulk KV append + causal sliding-window attention) for a plain
    prompt run (keys in flight, only in-window tokens get slots) and for a chunked-prefill run (every
    token stored, attention reads the paged cache); metadata is built once, outside the timed region."""
    res = {}
    g = torch.Generator(device=dev).manual_seed(0)
    T = S * L
    q = torch.randn(T, HQ, D, device=dev, dtype=torch.bfloat16, generator=g)
    k = torch.randn(T, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    v = torch.randn(T, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    out = torch.empty_like(q)
    visits = S * ((WL + 1) * (WL + 2) // 2 + (L - WL - 1) * (WL + 1))      # sum_i min(i + 1, window_left + 1)
    flops = 4 * HQ * D * visits
    impl = sb.MetaAttentionImpl(HQ, D, D ** -0.5, HKV, None, WL + 1, "auto")
    for name, chunked in (("prompt_inflight_kv", False), ("chunked_paged_kv", True)):
        nb = S * ((L if chunked else WL) // BS + 3) + 8
        runner = sb.SwaCacheRunner(1, nb, BS, WL, HKV, D, torch.bfloat16, dev, max_seqs=S, max_chunk_tokens=L)
        for s in range(S):
            runner.add_seq(s)
        t0 = time.perf_counter()
        meta = runner.build_step([(s, L) for s in range(S)], [], chunked_prefill=chunked)
        host_ms = (time.perf_counter() - t0) * 1e3
        stored = int((meta.slot_mapping >= 0).sum())

        def run():
            impl.forward(None, q, k, v, None, None, None, runner.kv_caches[0], meta, output=out)

        run()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        for a, b in evs:
            a.record()
            run()
            b.record()
        torch.cuda.synchronize()
        ms = statistics.median(a.elapsed_time(b) for a, b in evs)
        # the append alone
        eva = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        for a, b in eva:
            a.record()
            sb.ops.kv_append(k, v, runner.kv_caches[0][0], runner.kv_caches[0][1], meta.slot_mapping)
            b.record()
        torch.cuda.synchronize()
        ms_app = statistics.median(a.elapsed_time(b) for a, b in eva)
        app_bytes = stored * 2 * HKV * D * E * 2 + T * 8
        res[name] = {"ms_append_plus_attention": round(ms, 3), "ms_append": round(ms_app, 4),
                     "tokens_stored": stored, "append_GBps": round(app_bytes / (ms_app * 1e-3) / 1e9, 1),
                     "attention_TFLOPs": round(flops / ((ms - ms_app) * 1e-3) / 1e12, 1),
                     "mfma_frac_of_bf16_peak": round(flops / ((ms - ms_app) * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                     "prefill_tok_per_s_layer": round(T / (ms * 1e-3)), "host_metadata_ms": round(host_ms, 1)}
        del runner
    res["workload"] = f"BASELINE config 4: {S} x {L} new tokens, window_left {WL}, block_size {BS}, one layer"
    res["attention_flops"] = flops
    return res


def bench_decode_sweep(sb, dev, batches=(16, 32, 48, 64, 80, 96, 100, 128, 160, 192, 200, 256, 300, 384), iters=30):
    """Decode attention alone over batch sizes, every sequence window-saturated (8000 tokens, window_left
    4096): the split the library picks by itself (`auto`) next to the fixed and the balanced split forced,
    to show what the split policy buys at row counts that fit the 256 CUs badly."""
    rows = []
    lib = sb._native.lib()
    for B in batches:
        lens_t = torch.full((B,), 8000)
        lo_blk = torch.clamp((lens_t - 1 - WL) // BS, min=0)
        nblk = (lens_t - 1) // BS - lo_blk + 1
        nb = int(nblk.sum()) + 8
        g = torch.Generator().manual_seed(0)
        perm = torch.randperm(nb, generator=g)
        tables = torch.zeros(B, int(nblk.max()), dtype=torch.int32)
        p = 0
        for b in range(B):
            tables[b, :nblk[b]] = perm[p:p + int(nblk[b])]
            p += int(nblk[b])
        seqlens = (lens_t - lo_blk * BS).to(torch.int32)
        host_lens = seqlens.tolist()
        seqlens, tables = seqlens.to(dev), tables.to(dev)
        kvs = [torch.randn(2, nb, BS, HKV, D, device=dev, dtype=torch.bfloat16) for _ in range(2 if B > 64 else 4)]
        q = torch.randn(B, HQ, D, device=dev, dtype=torch.bfloat16)
        msl = max(host_lens)
        n_split = lib.sb_swa_decode_auto_split(B, HKV, msl, WL)
        row = {"rows": B, "n_split": n_split, "policy": "balanced" if sb.ops.prefer_balanced_split(host_lens, WL, n_split) else "fixed"}
        for mode in ("auto", "fixed", "balanced"):
            kw = {} if mode == "auto" else dict(balanced=(mode == "balanced"))

            def call(i):
                kv = kvs[i % len(kvs)]
                sb.ops.swa_decode_attention(q, kv[0], kv[1], seqlens, block_table=tables, window_left=WL,
                                            max_seq_len=msl, host_seq_lens=host_lens, **kw)
            for i in range(4):
                call(i)
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for i in range(iters):
                call(i)
            b.record()
            torch.cuda.synchronize()
            us = a.elapsed_time(b) / iters * 1e3
            row[mode + "_us"] = round(us, 1)
            row[mode + "_TBps"] = round(B * (WL + 1) * HKV * D * 2 * E / us / 1e6, 2)
        rows.append(row)
        del kvs
        torch.cuda.empty_cache()
    return rows


def bench_gla_step(sb, dev, B3=64, H3=28, iters=100):
    """BASELINE config 3: one GLA decode step for 64 sequences x 28 heads, fp32 state [B, H, 128, 128] updated
    in place; rotating over state copies larger than the on-die cache. HIP events on every launch's own dispatch."""
    g = torch.Generator().manual_seed(0)
    states = [(torch.randn(B3, H3, D, D, generator=g) * 0.02).to(dev) for _ in range(3)]
    q3, k3, v3 = (torch.randn(B3, H3, 1, D, generator=g).bfloat16().to(dev) for _ in range(3))
    g3 = (torch.nn.functional.logsigmoid(torch.randn(B3, H3, 1, D, generator=g)) / 16).to(dev)
    o3 = torch.empty(B3, H3, 1, D, dtype=torch.bfloat16, device=dev)
    for i in range(10):
        sb.ops.gla_recurrent(q3, k3, v3, g3, states[i % 3], None, None, o3)
    ev3 = [sb.ops.timing_events(dev) for _ in range(iters)]   # events on each kernel's own dispatch
    torch.cuda.synchronize()
    for i, pair in enumerate(ev3):
        sb.ops.gla_recurrent(q3, k3, v3, g3, states[i % 3], None, None, o3, profile_events=pair)
    torch.cuda.synchronize()
    ms3 = statistics.mean(a.elapsed_time(b) for a, b in ev3)
    bytes3 = 2 * B3 * H3 * D * D * 4 + B3 * H3 * (3 * D * 2 + D * 4 + D * 2)
    return {"workload": f"BASELINE config 3: B={B3}, H={H3}, fp32 state", "kernel": "gla_recurrent_kernel<f32 state, one step>",
            "kernel_ms": round(ms3, 4), "bytes_per_launch": bytes3, "GBps": round(bytes3 / (ms3 * 1e-3) / 1e9, 1),
            "frac_hbm_peak": round(bytes3 / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}


def bench_gla_prompt(sb, dev, S=16, L=8192, H=28, iters=3):
    """The GLA layers' share of BASELINE config 4 (16 prompts x 8192 tokens): one packed launch
    over token-major [tokens, H, D] projections, states read from and left in the slot cache.
    bf16 prompts run the recurrence 16 tokens at a time on the matrix cores; the step-by-step fp32
    vector kernel is timed beside it. Bytes: q, k, v, out in bf16 and the fp32 gate, once each."""
    g = torch.Generator().manual_seed(0)
    tokens = S * L
    q, k, v = (torch.randn(tokens, H, D, generator=g).bfloat16().to(dev) for _ in range(3))
    gate = (torch.nn.functional.logsigmoid(torch.randn(tokens, H, D, generator=g)) / 16).to(dev)
    cache = torch.zeros(S, H, D, D, device=dev)
    cu = torch.arange(0, tokens + 1, L, dtype=torch.int32, device=dev)
    slots = torch.arange(S, dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    times = {}
    for name, vector_only in (("matrix_cores", False), ("vector_only", True)):
        sb.ops.gla_recurrent_packed(q, k, v, gate, cache, cu, slots, out=out, max_seq_len=L, vector_only=vector_only)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        for a, b in evs:
            a.record()
            sb.ops.gla_recurrent_packed(q, k, v, gate, cache, cu, slots, out=out, max_seq_len=L, vector_only=vector_only)
            b.record()
        torch.cuda.synchronize()
        times[name] = statistics.mean(a.elapsed_time(b) for a, b in evs)
    ms = times["matrix_cores"]
    nbytes = tokens * H * D * (4 * 2 + 4) + 2 * S * H * D * D * 4
    return {"workload": f"GLA layer over BASELINE config 4's prompts: {S} x {L} tokens, H={H}, bf16 q/k/v, fp32 gate and state",
            "kernel": "gla_chunk_kernel", "kernel_ms": round(ms, 3), "prompt_tokens_per_s_layer": round(tokens / (ms * 1e-3), 0),
            "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "vector_only_kernel_ms": round(times["vector_only"], 3)}


def bench_gla_prompt_shared(sb, dev, H=28, Hk=4, iters=3):
    """The same 131 072 prompt tokens through a GLA layer that keeps one state per kv head (k, v and the gate with
    4 heads, q with 28), as 16 long and as 64 shorter prompts: one workgroup per query head (two ordered
    launches) against one workgroup per group of 7 query heads (one launch, the state advanced once)."""
    res = {"workload": f"GLA layer with one state per kv head, 131 072 prompt tokens, {H} q / {Hk} kv heads, bf16 q/k/v, fp32 gate and state"}
    for S, L in ((16, 8192), (64, 2048)):
        g = torch.Generator().manual_seed(0)
        tokens = S * L
        q = torch.randn(tokens, H, D, generator=g).bfloat16().to(dev)
        k, v = (torch.randn(tokens, Hk, D, generator=g).bfloat16().to(dev) for _ in range(2))
        gate = (torch.nn.functional.logsigmoid(torch.randn(tokens, Hk, D, generator=g)) / 16).to(dev)
        cache = torch.zeros(S, Hk, D, D, device=dev)
        cu = torch.arange(0, tokens + 1, L, dtype=torch.int32, device=dev)
        out = torch.empty_like(q)
        entry = {}
        for name, per_head in (("per_query_head_ms", True), ("per_group_ms", False), ("as_dispatched_ms", None)):
            sb.ops.gla_recurrent_packed(q, k, v, gate, cache, cu, out=out, max_seq_len=L, per_head=per_head)
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
            for a, b in evs:
                a.record()
                sb.ops.gla_recurrent_packed(q, k, v, gate, cache, cu, out=out, max_seq_len=L, per_head=per_head)
                b.record()
            torch.cuda.synchronize()
            entry[name] = round(statistics.mean(a.elapsed_time(b) for a, b in evs), 3)
        res[f"{S}x{L}"] = entry
    return res


def bench_hybrid(sb, dev, B=256, steps=128, warmup=4, kv_quant=None, gla_state_dtype=torch.float32,
                 gla_shared_states=False):
    """BASELINE config 5: the cache work of 128 consecutive decode steps of the 28-layer stack
    (14 GLA state layers + 14 paged SWA layers, one shared block table), B=256, every sequence at a
    logical context of 512k tokens (window-saturated), real appends, eviction and block recycling."""
    c = sb.HybridDecodeCache(B, randomize=True, device=dev, kv_quant=kv_quant, gla_state_dtype=gla_state_dtype,
                             gla_shared_states=gla_shared_states)
    c.start(512 * 1024)
    g = torch.Generator(device=dev).manual_seed(1)
    q = torch.randn(B, HQ, D, device=dev, dtype=torch.bfloat16, generator=g)
    k = torch.randn(B, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    v = torch.randn(B, HKV, D, device=dev, dtype=torch.bfloat16, generator=g)
    gh = c.gla_state_heads  # heads of the GLA k, v, gate: all 28, or the 4 kv heads with shared states
    gq = torch.randn(B, HQ, 1, D, device=dev, dtype=torch.bfloat16, generator=g)
    gk, gv = (torch.randn(B, gh, 1, D, device=dev, dtype=torch.bfloat16, generator=g) for _ in range(2))
    gg = torch.nn.functional.logsigmoid(torch.randn(B, gh, 1, D, device=dev, generator=g)) / 16
    out = torch.empty(B, HQ, D, device=dev, dtype=torch.bfloat16)

    def layers(meta):
        for li in range(c.num_layers):
            if li % 2 == 0:
                c.gla_layer(li, gq, gk, gv, gg)
            else:
                c.swa_layer(li, q, k, v, meta, out)

    host = []
    for _ in range(warmup):
        layers(c.step_metadata())
    torch.cuda.synchronize()
    c.host_wait_s = 0.0
    t0 = time.perf_counter()
    for _ in range(steps):
        th = time.perf_counter()
        meta = c.step_metadata()
        host.append(time.perf_counter() - th)
        layers(meta)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    # host work of a step's metadata: the time inside step_metadata() minus what it spent waiting for a pinned
    # staging set to come free (the host runs up to 4 steps ahead of the GPU, then waits for it)
    host_work_ms = (sum(host) - c.host_wait_s) / steps * 1e3
    gpu = []
    for _ in range(8):  # device time of one step with the host out of the way
        meta = c.step_metadata()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        layers(meta)
        b.record()
        torch.cuda.synchronize()
        gpu.append(a.elapsed_time(b))
    by = c.bytes_per_step()
    gpu_ms = statistics.median(gpu)
    res = {"workload": f"BASELINE config 5: 28-layer hybrid decode step, B={B}, logical context 512k, "
                       f"{steps} consecutive steps" + ({"int8": ", SWA K/V as per-row INT8", "fp8": ", SWA K/V as fp8 (e4m3fn)"}.get(kv_quant, ""))
                       + (", GLA state stored as bf16" if gla_state_dtype == torch.bfloat16 else "")
                       + (", one GLA state per kv head" if gla_shared_states else ""),
           "bytes_per_step": by,
           "host_stepped": {"ms_per_step": round(ms, 3), "decode_tok_per_s": round(B / (ms * 1e-3)),
                            "GBps": round(by / (ms * 1e-3) / 1e9, 1),
                            "frac_hbm_peak": round(by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                            "gpu_ms_per_step": round(gpu_ms, 3),
                            "host_metadata_ms_per_step": round(host_work_ms, 3),
                            "host_waiting_for_gpu_ms_per_step": round(c.host_wait_s / steps * 1e3, 3),
                            "step_minus_gpu_ms": round(max(0.0, ms - gpu_ms), 3)}}
    # the same steps with the block manager advanced on the device and the whole step (advance + 28
    # layers) replayed from one captured graph: no host work per step
    c.enable_device_advance()
    graph = c.capture_step(layers)
    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    gms = (time.perf_counter() - t0) / steps * 1e3
    c.device_state.check()
    res["graph_replayed"] = {"ms_per_step": round(gms, 3), "decode_tok_per_s": round(B / (gms * 1e-3)),
                             "GBps": round(by / (gms * 1e-3) / 1e9, 1),
                             "frac_hbm_peak": round(by / (gms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--n-split", type=int, default=0)
    ap.add_argument("--unfused", action="store_true", help="append with a separate kv_append launch")
    ap.add_argument("--force-valu", action="store_true",
                    help="run the vector-ALU split kernel instead of the matrix-core one (for comparison profiles)")
    ap.add_argument("--per-segment", action="store_true",
                    help="run the per-segment matrix-core split kernel instead of the stream kernel (for comparison profiles)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-hybrid", action="store_true", help="skip the 28-layer hybrid decode step (config 5) section")
    ap.add_argument("--extras", action="store_true", help="also time the GLA state update (config 3), chunked prefill (config 4) and the "
                                                    "28-layer hybrid decode step (config 5)")
    ap.add_argument("--only", choices=("prefill", "hybrid", "hybrid_int8", "hybrid_fp8", "hybrid_lean", "hybrid_shared",
                                       "hybrid_leanest", "gla_prompt", "gla_prompt_shared", "gla_step", "decode_sweep"), default=None,
                    help="run just that section and print its JSON (short runs for profiling one kernel)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import __graft_entry__ as entry
    sb = entry.load_package()
    sb._native.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.only == "prefill":
        print(json.dumps({"prefill": bench_prefill(sb, dev)}))
        return
    if args.only == "gla_prompt":
        print(json.dumps({"gla_prompt": bench_gla_prompt(sb, dev)}))
        return
    if args.only == "gla_prompt_shared":
        print(json.dumps({"gla_prompt_shared_states": bench_gla_prompt_shared(sb, dev)}))
        return
    if args.only == "gla_step":
        print(json.dumps({"gla_state_update": bench_gla_step(sb, dev), "gla_state_update_b256": bench_gla_step(sb, dev, B3=256, iters=40)}))
        return
    if args.only == "decode_sweep":
        print(json.dumps({"decode_sweep": bench_decode_sweep(sb, dev)}))
        return
    if args.only == "hybrid":
        print(json.dumps({"hybrid_decode": bench_hybrid(sb, dev, steps=min(args.steps, 128))}))
        return
    if args.only == "hybrid_lean":
        print(json.dumps({"hybrid_decode_int8_kv_bf16_state": bench_hybrid(
            sb, dev, steps=min(args.steps, 128), kv_quant="int8", gla_state_dtype=torch.bfloat16)}))
        return
    if args.only == "hybrid_shared":
        print(json.dumps({"hybrid_decode_shared_gla_states": bench_hybrid(
            sb, dev, steps=min(args.steps, 128), gla_shared_states=True)}))
        return
    if args.only == "hybrid_leanest":
        print(json.dumps({"hybrid_decode_fp8_kv_shared_gla_states": bench_hybrid(
            sb, dev, steps=min(args.steps, 128), kv_quant="fp8", gla_shared_states=True)}))
        return
    if args.only == "hybrid_fp8":
        print(json.dumps({"hybrid_decode_fp8_kv": bench_hybrid(sb, dev, steps=min(args.steps, 128), kv_quant="fp8")}))
        return
    if args.only == "hybrid_int8":
        print(json.dumps({"hybrid_decode_int8_kv": bench_hybrid(sb, dev, steps=min(args.steps, 128), kv_quant="int8")}))
        return

    # The CPU baseline runs first: the GPU sections then come in one block at the end of the run.
    cpu = None if args.no_cpu_baseline else cpu_baseline()

    prob = build_config2(dev)
    kv, n_copies = prob["kv"], len(prob["kv"])

    new_kv = dict(new_key=prob["k"], new_value=prob["v"], new_slot_mapping=prob["slots"])

    def attend(c, phases, **kw):
        sb.ops.swa_decode_attention(prob["q"], c[0], c[1], prob["seqlens"], block_table=prob["tables"],
                                    window_left=WL, out=prob["out"], max_seq_len=prob["max_seq_len"],
                                    n_split=args.n_split, phases=phases, force_valu=args.force_valu, balanced=False,
                                    per_segment=args.per_segment, **kw)

    def step(i, events=None):
        """One layer-step as MetaAttentionImpl.forward runs a pure decode batch: the split kernel
        appends each sequence's new K/V row at its slot and attends; the merge kernel follows.
        --unfused runs the append as a launch of its own (what mixed prefill/decode steps do).
        `events`: a (start, stop) pair of HIP events attached to the split kernel's own dispatch
        (hipExtLaunchKernel): they put no marker of their own into the stream."""
        c = kv[i % n_copies]
        kw = new_kv
        if args.unfused:
            sb.ops.kv_append(prob["k"], prob["v"], c[0], c[1], prob["slots"])
            kw = {}
        attend(c, 0, profile_events=events, **kw)

    n_split = args.n_split or sb._native.lib().sb_swa_decode_auto_split(prob["B"], HKV, prob["max_seq_len"], WL)
    # How the step is timed.
    #  * ramp: whatever --warmup says, RAMP_STEPS more untimed steps (>= 50 ms of the same GPU work) run right
    #    before the timed region, so the clocks are where a serving loop holds them (the CPU baseline and the
    #    set-up leave the GPU idle for seconds).
    #  * the timed region is `steps` steps, back to back, with nothing else in the stream: no events ride on its
    #    launches. It runs REGIONS times in a row, each between two synchronize() calls and timed by one pair of
    #    HIP events recorded on the stream around it. The start marker is recorded behind PRE_ROLL untimed steps
    #    of the same work, so that the first timed launch is already queued when the marker completes: on an
    #    empty queue the marker completes at once and the ~25 us the host then takes to issue the first launch
    #    are charged to the region (a 1-step region reads 112 us, a 200-step one 86.4 us per step). The line
    #    reports the median region; the same regions started on an empty queue, and their host-clock time from
    #    the first launch to the end of synchronize(), are given beside it.
    #  * the split kernel's own duration comes from a separate pass right after: KERNEL_SAMPLES steps whose
    #    split kernel carries a pair of HIP events on its own dispatch (hipExtLaunchKernel; the
    #    profile_*_event fields of sb_swa_decode_args). Such a launch delays the one behind it by about 6 us,
    #    which is why the pass is kept out of the timed region; the kernel's own interval is not affected.
    RAMP_STEPS, REGIONS, KERNEL_SAMPLES, PRE_ROLL = 640, 11, 64, 2
    timed = not args.force_valu
    for i in range(args.warmup):
        step(i)
    for i in range(RAMP_STEPS):
        step(i)
    torch.cuda.synchronize()

    def regions(pre_roll):
        by_events, by_host = [], []
        for _ in range(REGIONS):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            for i in range(pre_roll):
                step(i)
            a.record()
            for i in range(args.steps):
                step(i)
            b.record()
            torch.cuda.synchronize()
            by_host.append(time.perf_counter() - t0)
            by_events.append(a.elapsed_time(b) * 1e-3)
        return by_events, by_host

    idle_ev, idle_host = regions(0)
    region_ev, _ = regions(PRE_ROLL)
    wall = statistics.median(region_ev)
    ms_per_step = wall / args.steps * 1e3
    value = prob["bytes_step"] / (wall / args.steps) / 1e9
    if timed:
        evs = [sb.ops.timing_events(dev) for _ in range(KERNEL_SAMPLES)]
        for i, pair in enumerate(evs):
            step(i, pair)
        torch.cuda.synchronize()
    else:  # the vector-ALU comparison kernel has no timed launch: bracket its launches in a loop of their own
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(KERNEL_SAMPLES)]
        for i, (a, b) in enumerate(evs):
            a.record()
            attend(kv[i % n_copies], 1, **({} if args.unfused else new_kv))
            b.record()
            attend(kv[i % n_copies], 2)
        torch.cuda.synchronize()
    k_ms = statistics.mean(a.elapsed_time(b) for a, b in evs)
    achieved = prob["bytes_split_kernel"] / (k_ms * 1e-3) / 1e9

    default_workload = not (args.force_valu or args.unfused or args.n_split or args.per_segment)
    traffic, traffic_source = recorded_traffic() if default_workload else (None, "not the default workload")
    line = {
        "metric": "SWA decode-attn+append GB/s (% of HBM peak) and decode tok/s, 7B shapes, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE config 2: paged SWA decode, one layer-step (KV append + window attention)",
                   "batch": prob["B"], "q_heads": HQ, "kv_heads": HKV, "head_dim": D, "block_size": BS,
                   "window_left": WL, "context_lens": "U[1024,32768] seed 0", "n_split": int(n_split),
                   "kv_cache_copies_rotated": n_copies, "bytes_per_step": prob["bytes_step"]},
        "timing": {"ramp_steps": RAMP_STEPS, "regions": REGIONS, "region": f"{args.steps} steps back to back, no events on its launches",
                   "reported": f"median region, one HIP event pair on the stream around each region, start marker behind {PRE_ROLL} "
                               "untimed steps (queue not empty when the clock starts)",
                   "ms_per_step_regions_events": [round(t / args.steps * 1e3, 4) for t in region_ev],
                   "ms_per_step_median_started_on_empty_queue": round(statistics.median(idle_ev) / args.steps * 1e3, 4),
                   "ms_per_step_median_host_clock_empty_queue": round(statistics.median(idle_host) / args.steps * 1e3, 4)},
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "decode_tok_per_s_layer_step": round(prob["B"] / (wall / args.steps), 1),
        "roofline": {"bound": "hbm", "kernel": "swa_decode_split_kernel<BF16,7> (vector ALU)" if args.force_valu
                     else ("swa_decode_split_mfma_kernel<BF16>" if args.per_segment else "swa_decode_stream_kernel<BF16, fixed split>"), "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source, "kernel_ms": round(k_ms, 4),
                     "kernel_ms_measured": f"HIP events on the kernel's own dispatch, mean of {len(evs)} consecutive steps run right after the "
                                           "timed region (an event-carrying launch delays the next one by ~6 us, the kernel's own interval is unaffected)" if timed
                     else "HIP events around the launches of a second loop (kernel + dispatch latency)",
                     "bytes_per_launch": prob["bytes_split_kernel"]},
    }

    # plain streaming copy of 1 GiB in the same run: what this box's HBM gives a copy kernel
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        sb.ops.stream_copy(dst, src)
    evc = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(10)]
    for a, b in evc:
        a.record()
        sb.ops.stream_copy(dst, src)
        b.record()
    torch.cuda.synchronize()
    copy_ms = statistics.mean(a.elapsed_time(b) for a, b in evc)
    line["stream_copy_GBps_read_plus_write"] = round(2 * (1 << 30) / (copy_ms * 1e-3) / 1e9, 1)
    del src, dst

    if args.extras:
        line["gla_state_update"] = bench_gla_step(sb, dev)
        line["prefill"] = bench_prefill(sb, dev)
        torch.cuda.empty_cache()
        line["gla_prompt"] = bench_gla_prompt(sb, dev)
        line["gla_prompt_shared_states"] = bench_gla_prompt_shared(sb, dev)
        torch.cuda.empty_cache()
        line["hybrid_decode_int8_kv"] = bench_hybrid(sb, dev, kv_quant="int8")
        torch.cuda.empty_cache()
        line["hybrid_decode_fp8_kv"] = bench_hybrid(sb, dev, kv_quant="fp8")
        torch.cuda.empty_cache()
        # the storage formats of the reference's own variants: bf16 state cache (its serving path), INT8 K/V (W8ASpike)
        line["hybrid_decode_int8_kv_bf16_state"] = bench_hybrid(sb, dev, kv_quant="int8", gla_state_dtype=torch.bfloat16)
        torch.cuda.empty_cache()
        # one GLA state per kv head (same outputs, a seventh of the state traffic), alone and with fp8 K/V
        line["hybrid_decode_shared_gla_states"] = bench_hybrid(sb, dev, gla_shared_states=True)
        torch.cuda.empty_cache()
        line["hybrid_decode_fp8_kv_shared_gla_states"] = bench_hybrid(sb, dev, kv_quant="fp8", gla_shared_states=True)
        torch.cuda.empty_cache()

    # the metric's other half, decode tokens/s at 7B shapes: the whole 28-layer cache step (config 5)
    if not args.no_hybrid:
        torch.cuda.empty_cache()
        line["hybrid_decode"] = bench_hybrid(sb, dev)
        line["decode_tok_per_s_28_layers"] = line["hybrid_decode"]["graph_replayed"]["decode_tok_per_s"]
        torch.cuda.empty_cache()

    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line))


if __name__ == "__main__":
    main()
