"""Tensor-level wrappers over the C ABI: validate shapes the way the reference's callers expect,
then enqueue the HIP kernel on torch's current stream. No wrapper computes anything itself.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional, Tuple

import torch

from . import _native as N

PAD_SLOT_ID = -1

# Split-K scratch of the decode kernel. Outside stream capture: one buffer per (device, stream), grown on
# demand (calls on one stream are ordered, so they can share it; calls on different streams must not).
# Under stream capture: one buffer per capture, kept until `release_graph_workspace` is told that the graph
# is gone (an engine that re-captures per batch size calls it when it drops the old graph). A captured graph
# replays into the addresses recorded at capture time, so such a buffer must never be replaced, shrunk or handed
# back to the allocator by a later, larger request (the allocator could give the block to another tensor
# while every replay still writes and merges partials there).
_workspaces: Dict[Tuple[torch.device, int], torch.Tensor] = {}
_graph_workspaces: Dict[Tuple[torch.device, int], list] = {}


def _capture_id(dev: torch.device) -> int:
    """Sequence number of the stream capture torch's current stream is part of, 0 if none."""
    cid = C.c_uint64(0)
    N.check(N.lib().sb_stream_capture_id(N.stream_ptr(dev), C.byref(cid)), "stream_capture_id")
    return cid.value


_COUNTER_BYTES = 64 << 10   # arrival counters of the in-kernel merge at the head of a workspace: zero between launches


def _new_workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
    ws[:_COUNTER_BYTES].zero_()   # only the counters need a known start; partials are written before they are read
    return ws


def _workspace(dev: torch.device, nbytes: int) -> Optional[torch.Tensor]:
    if nbytes == 0:
        return None
    cap = _capture_id(dev)
    if cap:
        # (allocated inside the capture: the 64 KiB counter fill becomes a node of the graph and runs at every
        # replay, which is harmless: the counters are zero between launches anyway)
        owned = _graph_workspaces.setdefault((dev, cap), [])
        if not owned or owned[-1].numel() < nbytes:
            # (a smaller buffer handed out earlier in this capture stays in the list: earlier nodes use it)
            owned.append(_new_workspace(dev, nbytes))
        return owned[-1]
    key = (dev, N.stream_ptr(dev))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = _new_workspace(dev, nbytes)
        _workspaces[key] = ws
    return ws


def graph_workspace_ids(device=None):
    """Capture ids that still own split-K workspaces (one id per stream capture that ran a split decode call)."""
    return sorted(c for d, c in _graph_workspaces if device is None or d == torch.device(device))


def release_graph_workspace(capture_id: Optional[int] = None, device=None) -> int:
    """Drop the workspaces captured graphs own: those of one capture (`capture_id`, from
    `graph_workspace_ids()`), or all of them. Call it when the graph is destroyed, never while it may still be
    replayed: every replay writes its partial results there. Returns the bytes handed back to the allocator."""
    freed = 0
    for key in [k for k in _graph_workspaces
                if (capture_id is None or k[1] == capture_id) and (device is None or k[0] == torch.device(device))]:
        freed += sum(t.numel() for t in _graph_workspaces.pop(key))
    return freed


def _inner_contiguous(t: torch.Tensor, name: str) -> None:
    if t.stride(-1) != 1:
        raise ValueError(f"{name} must have a contiguous last dimension, got strides {t.stride()}")


def kv_append(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
              slot_mapping: torch.Tensor) -> None:
    """Scatter key/value [T, Hkv, D] into the paged caches [nb, bs, Hkv, D] at slot_mapping [T]
    (int64; negative = skip). Same contract as reshape_and_cache_flash at
    vllm_hymeta/attention/meta_attention.py:790-799 with an unquantised kv_cache_dtype."""
    dev = N.require_gpu(key, value, key_cache, value_cache, slot_mapping)
    if key.dim() != 3 or value.shape != key.shape:
        raise ValueError(f"key/value must both be [num_tokens, num_kv_heads, head_size], got {tuple(key.shape)} "
                         f"and {tuple(value.shape)}")
    if key_cache.dim() != 4 or value_cache.shape != key_cache.shape:
        raise ValueError("key_cache/value_cache must both be [num_blocks, block_size, num_kv_heads, head_size]")
    T, Hkv, D = key.shape
    nb, bs, Hc, Dc = key_cache.shape
    if (Hc, Dc) != (Hkv, D):
        raise ValueError(f"cache heads/head_size {(Hc, Dc)} do not match key {(Hkv, D)}")
    if not (key.dtype == value.dtype == key_cache.dtype == value_cache.dtype):
        raise ValueError("key, value and caches must share one dtype (quantised KV is not supported)")
    if slot_mapping.dtype != torch.int64:
        raise ValueError(f"slot_mapping must be int64, got {slot_mapping.dtype}")
    slot_mapping = slot_mapping.flatten()
    if slot_mapping.numel() < T:
        raise ValueError(f"slot_mapping has {slot_mapping.numel()} entries for {T} tokens")
    if not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.contiguous()
    for t, n in ((key, "key"), (value, "value"), (key_cache, "key_cache"), (value_cache, "value_cache")):
        _inner_contiguous(t, n)
    if key_cache.stride() != value_cache.stride():
        raise ValueError("key_cache and value_cache must have identical strides")
    a = N.KvAppendArgs(
        key=N.ptr(key), value=N.ptr(value), k_cache=N.ptr(key_cache), v_cache=N.ptr(value_cache),
        slot_mapping=N.ptr(slot_mapping), num_tokens=T, num_kv_heads=Hkv, head_size=D, block_size=bs,
        dtype=N.dtype_code(key.dtype),
        key_stride_token=key.stride(0), key_stride_head=key.stride(1),
        value_stride_token=value.stride(0), value_stride_head=value.stride(1),
        cache_stride_block=key_cache.stride(0), cache_stride_row=key_cache.stride(1),
        cache_stride_head=key_cache.stride(2), num_blocks=nb, stream=N.stream_ptr(dev))
    N.check(N.lib().sb_kv_append(C.byref(a)), "kv_append")


def swa_decode_attention(
    q: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    seq_lens: torch.Tensor,
    *,
    block_table: Optional[torch.Tensor] = None,
    kv_start: Optional[torch.Tensor] = None,
    row_seq: Optional[torch.Tensor] = None,
    key_lo: Optional[torch.Tensor] = None,
    kv_strides: Optional[Tuple[int, int, int]] = None,
    block_size: Optional[int] = None,
    num_kv_heads: Optional[int] = None,
    window_left: int = -1,
    scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    return_lse: bool = False,
    max_seq_len: Optional[int] = None,
    n_split: int = 0,
    phases: int = 0,
    force_valu: bool = False,
    merge_in_kernel: bool = False,
    per_segment: bool = False,
    balanced: Optional[bool] = None,
    host_seq_lens=None,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
    fp8_scales: Optional[Tuple[float, float]] = None,
    pipeline_depth: int = 0,
    new_key: Optional[torch.Tensor] = None,
    new_value: Optional[torch.Tensor] = None,
    new_slot_mapping: Optional[torch.Tensor] = None,
    meta_k: Optional[torch.Tensor] = None,
    meta_v: Optional[torch.Tensor] = None,
    profile_events=None,
    softcap: float = 0.0,
    alibi_slopes: Optional[torch.Tensor] = None,
    meta_bias: Optional[Tuple[int, int]] = None,
):
    """Single-query window attention for each row of q [R, Hq, D].

    softcap > 0: every scaled score x becomes softcap * tanh(x / softcap); alibi_slopes [Hq] fp32 (device):
    -slope[h] * (query position - key index) is added, the query sitting at the row's last key. Both in front
    of the mask, the cap first (what flash-attn does with the backend's logits_soft_cap / alibi_slopes).
    With meta rows the cap applies to their scores too and their ALiBi term is -slope[h] * |row0 + r + M - rows - j|
    for row r and meta row j, meta_bias = (row0, rows): the call's rows are queries row0 .. of the `rows` queries
    the reference stacks into one sequence for its second attention (fa_kernel_metatoken.py:169-188); default
    (0, R).

    profile_events: (start, stop) torch.cuda.Event pair made by `timing_events()`: attached to the split
    kernel's own dispatch, so start.elapsed_time(stop) is that kernel's duration alone (fixed-split
    matrix-core kernel only).

    meta_k/meta_v [M, Hkv, D]: meta (sink) tokens every row also attends to, unmasked, inside the same
    softmax (key2/value2 of vllm_hymeta/attention/fa_kernel_metatoken.py:110-194, there a second
    attention merged by log-sum-exp). Fixed split only; over a byte-code cache bf16/fp16 queries only.

    new_key/new_value [R, Hkv, D] + new_slot_mapping [R] int64 (all three or none): the newest key
    of each row (index seq_lens[r]-1) is taken from these tensors and stored into the paged cache
    at its slot by the same launch (append + attention fused; paged mode, one row per sequence).

    paged mode (block_table [S, max_blocks] int32): key_cache/value_cache are
    [num_blocks, block_size, Hkv, D] and strides are taken from them.
    dense mode (block_table None): key_cache/value_cache are any tensors whose element offset
    for (sequence s, key i, head h) is (kv_start[s] + i)*kv_strides[1] + h*kv_strides[2];
    kv_strides = (block, row, head) in elements and num_kv_heads must be given.
    The query of row r sits at key index seq_lens[r]-1 of sequence row_seq[r] (default r) and sees
    keys in [max(seq_lens[r]-1-window_left, key_lo[r]), seq_lens[r]-1].
    max_seq_len (a host int bounding seq_lens) only sizes the split; it defaults to a bound
    derived from the table/window shapes so that no device value is read back.
    phases: 0 = whole op; 1 = split kernel only, 2 = merge kernel only (profiling aid).
    force_valu: run bf16/fp16 on the vector-ALU split kernel instead of the matrix-core one.
    merge_in_kernel: the matrix-core fixed split merges its partial results itself (the last wavefront of a
    row to finish does it) instead of leaving them to the merge kernel; same bits, measured no faster.
    balanced: cut the chunks of all rows, laid end to end, into equal runs (one per CU) instead of
    cutting each row into n_split runs (bf16/fp16, <= 1024 rows): faster when the rows' lengths differ
    a lot, a little slower when they do not. Default: decided from host_seq_lens (the same numbers
    as seq_lens, as Python ints) when the caller has them, else off.
    k_scale, v_scale (fp32 [num_blocks, Hkv, block_size]): the caches are per-row INT8 codes as
    kv_append_int8 wrote them (paged mode, bf16/fp16 queries, append not fused).
    fp8_scales (k_scale, v_scale floats): the caches are fp8 (e4m3fn) codes as kv_append_fp8 wrote them
    (float8_e4m3fn or uint8 tensors), dequantised as code * scale; same restrictions."""
    dev = N.require_gpu(q, key_cache, value_cache, seq_lens, block_table, kv_start, row_seq, key_lo, out)
    if q.dim() != 3:
        raise ValueError(f"q must be [rows, num_heads, head_size], got {tuple(q.shape)}")
    R, Hq, D = q.shape
    _inner_contiguous(q, "q")
    fp8_kv = fp8_scales is not None
    int8_kv = k_scale is not None or v_scale is not None or fp8_kv     # byte-code caches
    if fp8_kv:
        if k_scale is not None or v_scale is not None or block_table is None:
            raise ValueError("the fp8 cache needs paged mode and takes fp8_scales instead of k_scale/v_scale")
        if key_cache.dtype not in (torch.float8_e4m3fn, torch.uint8) or value_cache.dtype != key_cache.dtype:
            raise ValueError("with fp8_scales the caches must be float8_e4m3fn (or uint8) tensors")
        if key_cache.dtype != torch.uint8:
            key_cache, value_cache = key_cache.view(torch.uint8), value_cache.view(torch.uint8)
    if int8_kv:
        if not fp8_kv:
            N.require_gpu(q, k_scale, v_scale)
            if k_scale is None or v_scale is None or block_table is None:
                raise ValueError("the INT8 cache needs k_scale, v_scale and paged mode")
            if key_cache.dtype != torch.int8 or value_cache.dtype != torch.int8:
                raise ValueError("with k_scale/v_scale the caches must be int8")
        if q.dtype not in (torch.bfloat16, torch.float16) or force_valu:
            raise NotImplementedError("the INT8 cache needs bf16 or fp16 queries on the matrix-core path")
        if new_key is not None or new_value is not None or new_slot_mapping is not None:
            raise NotImplementedError("no fused append into the INT8 cache: call kv_append_int8 first")
    elif key_cache.dtype != q.dtype or value_cache.dtype != q.dtype:
        raise ValueError("q and the caches must share one dtype")
    if block_table is not None:
        if key_cache.dim() != 4 or value_cache.shape != key_cache.shape:
            raise ValueError("paged caches must be [num_blocks, block_size, num_kv_heads, head_size]")
        if key_cache.stride() != value_cache.stride():
            raise ValueError("key_cache and value_cache must have identical strides")
        _inner_contiguous(key_cache, "key_cache")
        nb, bs, Hkv, Dc = key_cache.shape
        kv_strides = (key_cache.stride(0), key_cache.stride(1), key_cache.stride(2))
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
            raise ValueError("block_table must be a 2-D int32 tensor with contiguous rows")
        bt_stride = block_table.stride(0)
        bound = block_table.shape[1] * bs
        if int8_kv and not fp8_kv:
            for t, name in ((k_scale, "k_scale"), (v_scale, "v_scale")):
                if t.shape != (nb, Hkv, bs) or t.dtype != torch.float32 or not t.is_contiguous():
                    raise ValueError(f"{name} must be a contiguous float32 [num_blocks, num_kv_heads, block_size] tensor")
    else:
        if kv_strides is None or num_kv_heads is None:
            raise ValueError("dense mode needs kv_strides and num_kv_heads")
        Hkv, Dc, bs, bt_stride = num_kv_heads, D, 16, 0
        if kv_start is not None and (kv_start.dtype != torch.int64 or not kv_start.is_contiguous()):
            raise ValueError("kv_start must be a contiguous int64 tensor")
        bound = max_seq_len if max_seq_len is not None else (window_left + 1 if window_left >= 0 else 1 << 20)
    if Dc != D:
        raise ValueError(f"head_size mismatch: q {D}, cache {Dc}")
    for t, n in ((seq_lens, "seq_lens"), (row_seq, "row_seq"), (key_lo, "key_lo")):
        if t is not None and (t.dtype != torch.int32 or t.dim() != 1 or not t.is_contiguous() or t.numel() < R):
            raise ValueError(f"{n} must be a contiguous int32 vector with one entry per query row")
    if scale is None:
        scale = D ** -0.5
    if out is None:
        out = torch.empty((R, Hq, D), dtype=q.dtype, device=dev)
    else:
        if out.shape != q.shape or out.dtype != q.dtype:
            raise ValueError("out must match q in shape and dtype")
        _inner_contiguous(out, "out")
    lse = torch.empty((R, Hq), dtype=torch.float32, device=dev) if return_lse else None
    fused = {}
    if new_key is not None or new_value is not None or new_slot_mapping is not None:
        if new_key is None or new_value is None or new_slot_mapping is None:
            raise ValueError("new_key, new_value and new_slot_mapping go together")
        N.require_gpu(q, new_key, new_value, new_slot_mapping)
        if block_table is None or row_seq is not None:
            raise ValueError("fused append needs paged mode and one query row per sequence")
        if new_key.shape != (R, Hkv, D) or new_value.shape != (R, Hkv, D) or new_key.dtype != q.dtype \
                or new_value.dtype != q.dtype:
            raise ValueError(f"new_key/new_value must be [{R}, {Hkv}, {D}] of the cache dtype")
        _inner_contiguous(new_key, "new_key")
        _inner_contiguous(new_value, "new_value")
        if new_slot_mapping.dtype != torch.int64 or new_slot_mapping.numel() < R or not new_slot_mapping.is_contiguous():
            raise ValueError("new_slot_mapping must be a contiguous int64 vector with one entry per row")
        fused = dict(new_key=N.ptr(new_key), new_value=N.ptr(new_value), new_slot_mapping=N.ptr(new_slot_mapping),
                     new_key_stride_row=new_key.stride(0), new_key_stride_head=new_key.stride(1),
                     new_value_stride_row=new_value.stride(0), new_value_stride_head=new_value.stride(1))
    if meta_k is not None or meta_v is not None:
        if meta_k is None or meta_v is None:
            raise ValueError("meta_k and meta_v go together")
        N.require_gpu(q, meta_k, meta_v)
        if int8_kv and (force_valu or q.dtype not in (torch.bfloat16, torch.float16)):
            raise NotImplementedError("meta tokens over a byte-code cache need bf16/fp16 queries on the matrix-core kernel")
        if meta_k.dim() != 3 or meta_k.shape[1:] != (Hkv, D) or meta_v.shape != meta_k.shape or \
                meta_k.dtype != q.dtype or meta_v.dtype != q.dtype or meta_k.stride() != meta_v.stride():
            raise ValueError(f"meta_k and meta_v must be [meta_tokens, {Hkv}, {D}] of q's dtype with equal strides")
        _inner_contiguous(meta_k, "meta_k")
        if meta_k.shape[0] > 0:
            fused.update(meta_k=N.ptr(meta_k), meta_v=N.ptr(meta_v), meta_len=meta_k.shape[0],
                         meta_stride_row=meta_k.stride(0), meta_stride_head=meta_k.stride(1))
            balanced = False
    if max_seq_len is None:
        max_seq_len = bound
    if window_left >= 0:
        max_seq_len = max(1, max_seq_len)
    L = N.lib()
    auto_balance = balanced is None
    if n_split == 0:
        n_split = L.sb_swa_decode_auto_split(R, Hkv, int(max_seq_len), int(window_left))
    can_balance = (q.dtype in (torch.bfloat16, torch.float16) and not int8_kv and not force_valu and R <= 1024
                   and "meta_k" not in fused)
    if auto_balance:
        # from the rows' lengths when the caller has them on the host, else as if every row were as long as
        # max_seq_len (the balanced split adapts to the real lengths on the device either way)
        if not can_balance:
            balanced = False
        elif host_seq_lens is not None:
            balanced = prefer_balanced_split(host_seq_lens, window_left, n_split)
        else:
            key = (R, int(max_seq_len), int(window_left), int(n_split))
            balanced = _SHAPE_POLICY.get(key)
            if balanced is None:
                if len(_SHAPE_POLICY) >= 4096:   # lengths that grow step by step would fill it without end
                    _SHAPE_POLICY.clear()
                balanced = _SHAPE_POLICY[key] = prefer_balanced_split([int(max_seq_len)] * R, window_left, n_split)
    if balanced and can_balance and n_split < 2:
        n_split = 2  # the balanced split always goes through partial results and the merge
    ws_bytes = L.sb_swa_decode_workspace_bytes(R, Hq, D, n_split)
    ws = _workspace(dev, ws_bytes)
    a = N.SwaDecodeArgs(
        q=N.ptr(q), k_cache=N.ptr(key_cache), v_cache=N.ptr(value_cache), out=N.ptr(out), lse=N.ptr(lse),
        block_table=N.ptr(block_table), kv_start=N.ptr(kv_start), row_seq=N.ptr(row_seq),
        seq_lens=N.ptr(seq_lens), key_lo=N.ptr(key_lo),
        workspace=N.ptr(ws), workspace_bytes=0 if ws is None else ws.numel(),
        num_rows=R, num_q_heads=Hq, num_kv_heads=Hkv, head_size=D, block_size=bs,
        window_left=int(window_left), max_seq_len=int(min(max_seq_len, 2**31 - 1)), n_split=int(n_split),
        dtype=N.dtype_code(q.dtype), phases=int(phases),
        flags=(N.SB_DECODE_FORCE_VALU if force_valu else 0) | (N.SB_DECODE_BALANCED if balanced else 0)
        | (N.SB_DECODE_MERGE_IN_KERNEL if merge_in_kernel else 0) | (N.SB_DECODE_PER_SEGMENT if per_segment else 0)
        | ((int(pipeline_depth) & 7) << 4),
        scale=float(scale),
        q_stride_row=q.stride(0), q_stride_head=q.stride(1),
        out_stride_row=out.stride(0), out_stride_head=out.stride(1),
        kv_stride_block=kv_strides[0], kv_stride_row=kv_strides[1], kv_stride_head=kv_strides[2],
        block_table_stride=bt_stride, stream=N.stream_ptr(dev),
        k_scale=N.ptr(k_scale), v_scale=N.ptr(v_scale),
        kv_quant=N.SB_KV_FP8 if fp8_kv else (N.SB_KV_INT8 if int8_kv else N.SB_KV_NONE),
        k_scale_tensor=float(fp8_scales[0]) if fp8_kv else 0.0, v_scale_tensor=float(fp8_scales[1]) if fp8_kv else 0.0,
        softcap=float(softcap), alibi_slopes=N.ptr(_slopes(alibi_slopes, Hq, dev)),
        meta_bias_row0=int(meta_bias[0]) if meta_bias else 0, meta_bias_rows=int(meta_bias[1]) if meta_bias else 0,
        **fused, **_event_args(profile_events))
    N.check(L.sb_swa_decode(C.byref(a)), "swa_decode")
    return (out, lse) if return_lse else out


def _slopes(alibi_slopes, num_q_heads: int, device) -> Optional[torch.Tensor]:
    """ALiBi slopes as the kernels read them: fp32 [Hq], contiguous, on the queries' device."""
    if alibi_slopes is None:
        return None
    t = torch.as_tensor(alibi_slopes, dtype=torch.float32, device=device).contiguous()
    if t.shape != (num_q_heads,):
        raise ValueError(f"alibi_slopes must have one slope per query head ({num_q_heads}), got {tuple(t.shape)}")
    return t


def timing_events(device) -> Tuple[torch.cuda.Event, torch.cuda.Event]:
    """A (start, stop) pair of timing events whose runtime handles exist already (torch creates the handle at
    the first record), to be handed to a kernel launch through `profile_events`."""
    pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    with torch.cuda.device(device):
        for e in pair:
            e.record()
    return pair


def _event_args(profile_events) -> dict:
    if profile_events is None:
        return {}
    start, stop = profile_events
    return dict(profile_start_event=start.cuda_event, profile_stop_event=stop.cuda_event)


def alloc_int8_kv_cache(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int, device):
    """(kv int8 [2, num_blocks, block_size, Hkv, D], scales fp32 [2, num_blocks, Hkv, block_size]),
    zero-filled: the paged K/V cache in its per-row INT8 form."""
    kv = torch.zeros((2, num_blocks, block_size, num_kv_heads, head_size), dtype=torch.int8, device=device)
    scales = torch.zeros((2, num_blocks, num_kv_heads, block_size), dtype=torch.float32, device=device)
    return kv, scales


def kv_append_int8(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   k_scale: torch.Tensor, v_scale: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """Quantise this step's K/V rows (per row: 128 signed bytes + one fp32 scale) and store them at
    their slots; slots < 0 are skipped. Caches int8 [nb, bs, Hkv, 128], scales fp32 [nb, Hkv, bs]."""
    dev = N.require_gpu(key, value, k_cache, v_cache, k_scale, v_scale, slot_mapping)
    if key.dim() != 3 or value.shape != key.shape or value.dtype != key.dtype:
        raise ValueError("key and value must be [tokens, num_kv_heads, head_size] of one dtype")
    T, Hkv, D = key.shape
    if k_cache.dtype != torch.int8 or v_cache.dtype != torch.int8 or k_cache.dim() != 4 or v_cache.shape != k_cache.shape \
            or k_cache.stride() != v_cache.stride():
        raise ValueError("k_cache and v_cache must be int8 [num_blocks, block_size, num_kv_heads, head_size] with equal strides")
    nb, bs = k_cache.shape[0], k_cache.shape[1]
    if k_cache.shape[2:] != (Hkv, D) or k_cache.stride(3) != 1:
        raise ValueError(f"cache rows must be [{Hkv}, {D}] with a contiguous head dimension")
    for t, name in ((k_scale, "k_scale"), (v_scale, "v_scale")):
        if t.shape != (nb, Hkv, bs) or t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous float32 [num_blocks, num_kv_heads, block_size] tensor")
    _inner_contiguous(key, "key")
    _inner_contiguous(value, "value")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous() or slot_mapping.numel() < T:
        raise ValueError("slot_mapping must be a contiguous int64 vector with one entry per token")
    a = N.KvAppendInt8Args(
        key=N.ptr(key), value=N.ptr(value), k_cache=N.ptr(k_cache), v_cache=N.ptr(v_cache),
        k_scale=N.ptr(k_scale), v_scale=N.ptr(v_scale), slot_mapping=N.ptr(slot_mapping), num_tokens=T,
        num_kv_heads=Hkv, head_size=D, block_size=bs, dtype=N.dtype_code(key.dtype),
        key_stride_token=key.stride(0), key_stride_head=key.stride(1),
        value_stride_token=value.stride(0), value_stride_head=value.stride(1),
        cache_stride_block=k_cache.stride(0), cache_stride_row=k_cache.stride(1), cache_stride_head=k_cache.stride(2),
        stream=N.stream_ptr(dev))
    N.check(N.lib().sb_kv_append_int8(C.byref(a)), "kv_append_int8")


def kv_append_fp8(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor, k_scale: float = 1.0, v_scale: float = 1.0) -> None:
    """Store this step's K/V rows as fp8 (e4m3fn) codes of x / scale (saturating at +-448) at their slots;
    slots < 0 are skipped. Caches float8_e4m3fn or uint8 [nb, bs, Hkv, 128]."""
    dev = N.require_gpu(key, value, k_cache, v_cache, slot_mapping)
    if key.dim() != 3 or value.shape != key.shape or value.dtype != key.dtype:
        raise ValueError("key and value must be [tokens, num_kv_heads, head_size] of one dtype")
    T, Hkv, D = key.shape
    if k_cache.dtype not in (torch.float8_e4m3fn, torch.uint8) or v_cache.dtype != k_cache.dtype or k_cache.dim() != 4 \
            or v_cache.shape != k_cache.shape or k_cache.stride() != v_cache.stride():
        raise ValueError("k_cache and v_cache must be float8_e4m3fn/uint8 [num_blocks, block_size, num_kv_heads, head_size] "
                         "with equal strides")
    if k_cache.shape[2:] != (Hkv, D) or k_cache.stride(3) != 1:
        raise ValueError(f"cache rows must be [{Hkv}, {D}] with a contiguous head dimension")
    _inner_contiguous(key, "key")
    _inner_contiguous(value, "value")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous() or slot_mapping.numel() < T:
        raise ValueError("slot_mapping must be a contiguous int64 vector with one entry per token")
    a = N.KvAppendFp8Args(
        key=N.ptr(key), value=N.ptr(value), k_cache=N.ptr(k_cache), v_cache=N.ptr(v_cache),
        slot_mapping=N.ptr(slot_mapping), num_tokens=T, num_kv_heads=Hkv, head_size=D, block_size=k_cache.shape[1],
        dtype=N.dtype_code(key.dtype), key_stride_token=key.stride(0), key_stride_head=key.stride(1),
        value_stride_token=value.stride(0), value_stride_head=value.stride(1),
        cache_stride_block=k_cache.stride(0), cache_stride_row=k_cache.stride(1), cache_stride_head=k_cache.stride(2),
        k_scale=float(k_scale), v_scale=float(v_scale), stream=N.stream_ptr(dev))
    N.check(N.lib().sb_kv_append_fp8(C.byref(a)), "kv_append_fp8")


def fp8_round(x: torch.Tensor, scale: float = 1.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x after a round trip through fp8: e4m3fn(clamp(x / scale, -448, 448)) * scale in x's dtype (what
    scaled_fp8_quant followed by the kernel's descale makes of a query, meta_attention.py:806-811).
    x: any shape with a contiguous last dimension that is a multiple of 8; out may be x."""
    dev = N.require_gpu(x, out)
    if x.dim() < 1 or x.stride(-1) != 1 or x.shape[-1] % 8 != 0:
        raise ValueError("x needs a contiguous last dimension that is a multiple of 8")
    x2 = x.reshape(-1, x.shape[-1]) if x.is_contiguous() else None
    if x2 is None:
        raise ValueError("x must be contiguous")
    if out is None:
        out = torch.empty_like(x)
    elif out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous():
        raise ValueError("out must be contiguous and match x in shape and dtype")
    N.check(N.lib().sb_fp8_round(N.ptr(x), N.ptr(out), x2.shape[0], x2.shape[1], x2.stride(0), x2.stride(0),
                                 N.dtype_code(x.dtype), float(scale), N.stream_ptr(dev)), "fp8_round")
    return out


def quantize_sym(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """quantize_sym of W8ASpike/window_attention.py:227-237 on x [rows, heads, 128]: every row replaced
    by its INT8 codes times its scale, rounded to x's dtype. out may be x."""
    dev = N.require_gpu(x, out)
    if x.dim() != 3:
        raise ValueError("x must be [rows, heads, head_size]")
    _inner_contiguous(x, "x")
    if out is None:
        out = torch.empty_like(x)
    elif out.shape != x.shape or out.dtype != x.dtype:
        raise ValueError("out must match x in shape and dtype")
    _inner_contiguous(out, "out")
    a = N.QuantizeSymArgs(in_=N.ptr(x), out=N.ptr(out), rows=x.shape[0], heads=x.shape[1], head_size=x.shape[2],
                          dtype=N.dtype_code(x.dtype), in_stride_row=x.stride(0), in_stride_head=x.stride(1),
                          out_stride_row=out.stride(0), out_stride_head=out.stride(1), stream=N.stream_ptr(dev))
    N.check(N.lib().sb_quantize_sym(C.byref(a)), "quantize_sym")
    return out


_SHAPE_POLICY: dict = {}  # (rows, max_seq_len, window_left, n_split) -> balanced, for calls without host lengths


def prefer_balanced_split(host_seq_lens, window_left: int, n_split: int) -> bool:
    """Whether the balanced split is expected to beat the fixed one for rows of these lengths
    (host ints; no device access)."""
    n = len(host_seq_lens)
    if n == 0 or n_split < 1:
        return False
    arr = (C.c_int32 * n)(*[int(x) for x in host_seq_lens])
    return bool(N.lib().sb_swa_decode_prefer_balanced(arr, n, int(window_left), int(n_split)))


def plan_decode_split(num_rows: int, num_kv_heads: int, max_seq_len: int, window_left: int, host_seq_lens) -> bool:
    """The `balanced` choice swa_decode_attention would make for this step, for callers that run
    many layers on the same lengths and want to decide once."""
    n_split = N.lib().sb_swa_decode_auto_split(int(num_rows), int(num_kv_heads), int(max_seq_len), int(window_left))
    return prefer_balanced_split(host_seq_lens, window_left, n_split)


PREFILL_TILE = 64  # query tokens per workgroup of the prefill kernel


class PrefillPlan:
    """Device-side description of one prefill launch: per-sequence query offsets and key counts, and
    the cover of the query axis by 64-token tiles. Built on the host from the step's length lists
    (which the scheduler already has as Python ints), uploaded with one copy."""

    __slots__ = ("cu_seqlens_q", "seq_lens_k", "tile_seq", "tile_q0", "num_tiles", "total_q", "num_seqs", "max_k",
                 "total_k")

    def __init__(self, query_lens, seq_lens_k, device):
        query_lens = [int(x) for x in query_lens]
        seq_lens_k = query_lens if seq_lens_k is None else [int(x) for x in seq_lens_k]
        if len(seq_lens_k) != len(query_lens):
            raise ValueError("query_lens and seq_lens_k must have one entry per sequence")
        cu, tile_seq, tile_q0 = [0], [], []
        for s, (lq, lk) in enumerate(zip(query_lens, seq_lens_k)):
            if lq < 0 or lk < lq:
                raise ValueError(f"sequence {s}: {lq} queries need at least as many keys, got {lk}")
            cu.append(cu[-1] + lq)
            for q0 in range(0, lq, PREFILL_TILE):
                tile_seq.append(s)
                tile_q0.append(q0)
        S, T = len(query_lens), len(tile_seq)
        packed = torch.tensor(cu + seq_lens_k + tile_seq + tile_q0, dtype=torch.int32).to(device, non_blocking=False)
        self.cu_seqlens_q = packed[:S + 1]
        self.seq_lens_k = packed[S + 1:2 * S + 1]
        self.tile_seq = packed[2 * S + 1:2 * S + 1 + T]
        self.tile_q0 = packed[2 * S + 1 + T:]
        self.num_tiles, self.total_q, self.num_seqs = T, cu[-1], S
        self.max_k, self.total_k = max(seq_lens_k, default=0), sum(seq_lens_k)


def swa_prefill_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    query_lens=None,
    seq_lens_k=None,
    plan: Optional[PrefillPlan] = None,
    block_table: Optional[torch.Tensor] = None,
    kv_start: Optional[torch.Tensor] = None,
    key_lo: Optional[torch.Tensor] = None,
    kv_strides: Optional[Tuple[int, int]] = None,
    num_kv_heads: Optional[int] = None,
    window_left: int = -1,
    scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    return_lse: bool = False,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
    fp8_scales: Optional[Tuple[float, float]] = None,
    meta_k: Optional[torch.Tensor] = None,
    meta_v: Optional[torch.Tensor] = None,
    softcap: float = 0.0,
    alibi_slopes: Optional[torch.Tensor] = None,
    meta_bias: Optional[Tuple[int, int]] = None,
):
    """Causal sliding-window attention for q [total_q, Hq, D] packed sequence after sequence.
    softcap / alibi_slopes: as for swa_decode_attention; query j of a sequence sits at key position
    seq_len_k - query_len + j. With meta rows: meta_bias = (row0, rows) as there (default (0, total_q)).
    With return_lse also the fp32 [total_q, Hq] natural-log log-sum-exp of each query's scores.
    meta_k/meta_v [M, Hkv, D]: meta (sink) tokens every query also attends to, unmasked, in the same
    softmax (not over byte-code caches).

    query_lens / seq_lens_k: per-sequence host ints (keys default to the queries: plain prompt), or a
    prebuilt `plan`. Query j of a sequence sits at key position seq_len_k - query_len + j.
    paged (block_table [S, max_blocks] int32): k/v are the caches [num_blocks, block_size, Hkv, D].
    dense (block_table None): k/v are [rows, Hkv, D]; keys of sequence s start at row kv_start[s]
    (int64 device vector; default: the same packing as q, which needs seq_lens_k == query_lens).
    With kv_strides = (row, head) in elements (and num_kv_heads), k/v may be any tensors whose
    element offset for (sequence s, key i, head h) is (kv_start[s] + i)*row + h*head.
    key_lo [S] int32: keys below key_lo[s] are invisible (left padding); a query that sees no key
    gets zeros.
    k_scale/v_scale (INT8 codes) or fp8_scales (e4m3fn codes): the paged caches are byte codes as
    kv_append_int8 / kv_append_fp8 wrote them; rows are dequantised on their way into the kernel."""
    dev = N.require_gpu(q, k, v, block_table, kv_start, key_lo, out, k_scale, v_scale)
    kv_quant = N.SB_KV_NONE
    if fp8_scales is not None:
        if block_table is None or k.dtype not in (torch.float8_e4m3fn, torch.uint8) or v.dtype != k.dtype:
            raise ValueError("fp8_scales needs paged float8_e4m3fn (or uint8) caches")
        if k.dtype != torch.uint8:
            k, v = k.view(torch.uint8), v.view(torch.uint8)
        kv_quant = N.SB_KV_FP8
    elif k_scale is not None or v_scale is not None:
        if k_scale is None or v_scale is None or block_table is None or k.dtype != torch.int8 or v.dtype != torch.int8:
            raise ValueError("k_scale and v_scale go together, with paged int8 caches")
        kv_quant = N.SB_KV_INT8
    if q.dim() != 3:
        raise ValueError(f"q must be [total_q, num_heads, head_size], got {tuple(q.shape)}")
    Tq, Hq, D = q.shape
    _inner_contiguous(q, "q")
    if kv_quant == N.SB_KV_NONE and (k.dtype != q.dtype or v.dtype != q.dtype):
        raise ValueError("q, k and v must share one dtype")
    if plan is None:
        if query_lens is None:
            raise ValueError("give query_lens (and seq_lens_k) or a prebuilt plan")
        plan = PrefillPlan(query_lens, seq_lens_k, dev)
    if plan.total_q != Tq:
        raise ValueError(f"query_lens sum to {plan.total_q}, q has {Tq} rows")
    if k.shape != v.shape or k.stride() != v.stride():
        raise ValueError("k and v must have identical shapes and strides")
    _inner_contiguous(k, "k")
    if block_table is not None:
        if k.dim() != 4:
            raise ValueError("paged caches must be [num_blocks, block_size, num_kv_heads, head_size]")
        nb, bs, Hkv, Dc = k.shape
        strides = (k.stride(0), k.stride(1), k.stride(2))
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1 \
                or block_table.shape[0] < plan.num_seqs:
            raise ValueError("block_table must be a 2-D int32 tensor with contiguous rows, one per sequence")
        if block_table.shape[1] * bs < plan.max_k:
            raise ValueError(f"block_table rows hold {block_table.shape[1] * bs} keys, a sequence has {plan.max_k}")
        if kv_quant == N.SB_KV_INT8:
            for t, name in ((k_scale, "k_scale"), (v_scale, "v_scale")):
                if t.shape != (nb, Hkv, bs) or t.dtype != torch.float32 or not t.is_contiguous():
                    raise ValueError(f"{name} must be a contiguous float32 [num_blocks, num_kv_heads, block_size] tensor")
        bt_stride = block_table.stride(0)
    else:
        bs, bt_stride = 16, 0
        if kv_strides is not None:
            if num_kv_heads is None or kv_start is None:
                raise ValueError("kv_strides needs num_kv_heads and kv_start")
            Hkv, Dc = num_kv_heads, k.shape[-1]
            strides = (0, int(kv_strides[0]), int(kv_strides[1]))
        else:
            if k.dim() != 3:
                raise ValueError("dense k/v must be [rows, num_kv_heads, head_size]")
            Hkv, Dc = k.shape[1], k.shape[2]
            strides = (0, k.stride(0), k.stride(1))
            if kv_start is None:
                if plan.total_k > k.shape[0]:
                    raise ValueError(f"k has {k.shape[0]} rows, the sequences hold {plan.total_k} keys")
                kv_start = plan.cu_seqlens_q.to(torch.int64)
        if kv_start.dtype != torch.int64 or not kv_start.is_contiguous() or kv_start.numel() < plan.num_seqs:
            raise ValueError("kv_start must be a contiguous int64 vector with one entry per sequence")
    if num_kv_heads is not None and num_kv_heads != Hkv:
        raise ValueError(f"num_kv_heads {num_kv_heads} does not match k's {Hkv}")
    if Dc != D:
        raise ValueError(f"head_size mismatch: q {D}, k {Dc}")
    if key_lo is not None and (key_lo.dtype != torch.int32 or not key_lo.is_contiguous()
                               or key_lo.numel() < plan.num_seqs):
        raise ValueError("key_lo must be a contiguous int32 vector with one entry per sequence")
    if scale is None:
        scale = D ** -0.5
    if out is None:
        out = torch.empty((Tq, Hq, D), dtype=q.dtype, device=dev)
    else:
        if out.shape != q.shape or out.dtype != q.dtype:
            raise ValueError("out must match q in shape and dtype")
        _inner_contiguous(out, "out")
    lse = torch.full((Tq, Hq), float("-inf"), dtype=torch.float32, device=dev) if return_lse else None
    if plan.num_tiles == 0:
        return (out, lse) if return_lse else out
    meta = {}
    if meta_k is not None or meta_v is not None:
        if meta_k is None or meta_v is None:
            raise ValueError("meta_k and meta_v go together")
        N.require_gpu(q, meta_k, meta_v)
        if meta_k.dim() != 3 or meta_k.shape[1:] != (Hkv, D) or meta_v.shape != meta_k.shape or \
                meta_k.dtype != q.dtype or meta_v.dtype != q.dtype or meta_k.stride() != meta_v.stride():
            raise ValueError(f"meta_k and meta_v must be [meta_tokens, {Hkv}, {D}] of q's dtype with equal strides")
        _inner_contiguous(meta_k, "meta_k")
        if meta_k.shape[0] > 0:
            meta = dict(meta_k=N.ptr(meta_k), meta_v=N.ptr(meta_v), meta_len=meta_k.shape[0],
                        meta_stride_row=meta_k.stride(0), meta_stride_head=meta_k.stride(1))
    a = N.SwaPrefillArgs(
        q=N.ptr(q), k=N.ptr(k), v=N.ptr(v), out=N.ptr(out),
        block_table=N.ptr(block_table), kv_start=N.ptr(kv_start) if block_table is None else None,
        key_lo=N.ptr(key_lo), cu_seqlens_q=N.ptr(plan.cu_seqlens_q), seq_lens_k=N.ptr(plan.seq_lens_k),
        tile_seq=N.ptr(plan.tile_seq), tile_q0=N.ptr(plan.tile_q0), num_tiles=plan.num_tiles,
        num_q_heads=Hq, num_kv_heads=Hkv, head_size=D, block_size=bs, window_left=int(window_left),
        dtype=N.dtype_code(q.dtype), scale=float(scale),
        q_stride_row=q.stride(0), q_stride_head=q.stride(1),
        out_stride_row=out.stride(0), out_stride_head=out.stride(1),
        kv_stride_block=strides[0], kv_stride_row=strides[1], kv_stride_head=strides[2],
        block_table_stride=bt_stride, stream=N.stream_ptr(dev), lse=N.ptr(lse),
        k_scale=N.ptr(k_scale), v_scale=N.ptr(v_scale), kv_quant=kv_quant,
        k_scale_tensor=float(fp8_scales[0]) if fp8_scales is not None else 0.0,
        v_scale_tensor=float(fp8_scales[1]) if fp8_scales is not None else 0.0,
        softcap=float(softcap), alibi_slopes=N.ptr(_slopes(alibi_slopes, Hq, dev)),
        meta_bias_row0=int(meta_bias[0]) if meta_bias else 0,
        meta_bias_rows=int(meta_bias[1]) if meta_bias else int(q.shape[0]), **meta)
    N.check(N.lib().sb_swa_prefill(C.byref(a)), "swa_prefill")
    return (out, lse) if return_lse else out


def lse_merge(out: torch.Tensor, lse: torch.Tensor, block_out: torch.Tensor, block_lse: torch.Tensor) -> None:
    """In place: (out, lse) becomes the attention over the union of the key sets behind (out, lse)
    and (block_out, block_lse). out/block_out [rows, H, D]; lse/block_lse fp32 [rows, H], natural log."""
    dev = N.require_gpu(out, lse, block_out, block_lse)
    if out.dim() != 3 or block_out.shape != out.shape or block_out.dtype != out.dtype:
        raise ValueError("out and block_out must be [rows, heads, head_size] of one dtype")
    R, H, D = out.shape
    for t, name in ((lse, "lse"), (block_lse, "block_lse")):
        if t.shape != (R, H) or t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous float32 [rows, heads] tensor")
    _inner_contiguous(out, "out")
    _inner_contiguous(block_out, "block_out")
    a = N.LseMergeArgs(out=N.ptr(out), lse=N.ptr(lse), block_out=N.ptr(block_out), block_lse=N.ptr(block_lse),
                       rows=R, heads=H, head_size=D, dtype=N.dtype_code(out.dtype),
                       out_stride_row=out.stride(0), out_stride_head=out.stride(1),
                       block_out_stride_row=block_out.stride(0), block_out_stride_head=block_out.stride(1),
                       stream=N.stream_ptr(dev))
    N.check(N.lib().sb_lse_merge(C.byref(a)), "lse_merge")


def meta_token_attention(q: torch.Tensor, k2: torch.Tensor, v2: torch.Tensor, scale: Optional[float] = None,
                         softcap: float = 0.0, alibi_slopes: Optional[torch.Tensor] = None,
                         meta_bias: Optional[Tuple[int, int]] = None):
    """Non-causal attention of every query row over the same few cached meta tokens
    (k2, v2 [M, Hkv, D]), as the second attention of fa_kernel_metatoken.py:174-188 / 261-275.
    Returns (out [rows, Hq, D], lse fp32 [rows, Hq]). Runs on the single-query kernel: every row is
    a query at position M-1 of one shared dense sequence. With softcap / alibi_slopes the rows are queries with
    an empty window that take the meta rows into their softmax; meta_bias = (row0, rows) places them in the
    reference's stacked sequence (see swa_decode_attention)."""
    dev = N.require_gpu(q, k2, v2)
    R = q.shape[0]
    M, Hkv, D = k2.shape
    if v2.shape != k2.shape or k2.dtype != q.dtype or v2.dtype != q.dtype:
        raise ValueError("k2 and v2 must be [meta_tokens, num_kv_heads, head_size] of q's dtype")
    _inner_contiguous(k2, "k2")
    _inner_contiguous(v2, "v2")
    if k2.stride() != v2.stride():
        raise ValueError("k2 and v2 must share their strides")
    zeros32 = torch.zeros(R, dtype=torch.int32, device=dev)
    if softcap > 0 or alibi_slopes is not None:
        # no window keys at all (a dense dummy sequence of length 0): the meta rows are the whole softmax
        return swa_decode_attention(
            q, k2, v2, zeros32, kv_start=torch.zeros(1, dtype=torch.int64, device=dev), row_seq=zeros32,
            kv_strides=(0, k2.stride(0), k2.stride(1)), num_kv_heads=Hkv, window_left=-1, scale=scale,
            return_lse=True, max_seq_len=1, n_split=1, balanced=False, meta_k=k2, meta_v=v2, softcap=softcap,
            alibi_slopes=alibi_slopes, meta_bias=meta_bias)
    return swa_decode_attention(
        q, k2, v2, torch.full((R,), M, dtype=torch.int32, device=dev), kv_start=torch.zeros(1, dtype=torch.int64, device=dev),
        row_seq=zeros32, kv_strides=(0, k2.stride(0), k2.stride(1)), num_kv_heads=Hkv, window_left=-1, scale=scale,
        return_lse=True, max_seq_len=M, n_split=1)


def gla_gate_range_hits(reset: bool = False) -> int:
    """How often the matrix-core GLA launches made with check_gates=True on the current device met gates beyond the block form's range (a
    pair of 16-token blocks whose log-gates sum below -80 for some key dim: results there under-weight
    near-diagonal terms; `vector_only=True` has no such limit) since the counter was last cleared: one count per
    prompt, head, 32 key dims and pair of blocks concerned. Waits for the device."""
    hits = C.c_int64(0)
    N.check(N.lib().sb_gla_gate_range_hits(C.byref(hits), 1 if reset else 0), "gla_gate_range_hits")
    return int(hits.value)


def gla_recurrent(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
                  slot_idx: Optional[torch.Tensor] = None, scale: Optional[float] = None,
                  out: Optional[torch.Tensor] = None, vector_only: bool = False, profile_events=None,
                  check_gates: bool = False, per_head: Optional[bool] = None) -> torch.Tensor:
    """q, k, v, g [B, H, T, D] (any batch/head/time strides, contiguous D); state
    [slots, H, D, D] fp32 or bf16, updated in place; returns o [B, H, T, D] in q's dtype.
    Rows with slot_idx == -1 are skipped (state and output untouched).
    Calls of 32 steps or more with bf16 q/k/v run 16 tokens at a time on the matrix cores (state, gates
    and accumulation in fp32, bf16 operand rounding on the output path); vector_only=True keeps them on
    the step-by-step fp32 kernel. check_gates=True: the block form counts gates beyond its range (see
    gla_gate_range_hits). per_head (shared states, block form): True = one workgroup per query head, False = one
    per group of query heads (the state advanced once for the group), None = chosen by the number of groups; the
    results are the same bits either way.
    Shared states: k, v, g may come with Hkv < H heads (H a multiple of Hkv, up to 8 query heads per kv
    head) and state as [slots, Hkv, D, D]: query head h then works on head h // (H // Hkv) of them, which is
    the reference's repeat_kv of k, v and the gate (hf_7B_model/gla_attention.py:147-149) without the
    copies, and every state crosses HBM once per step for its whole group."""
    dev = N.require_gpu(q, k, v, g, state, slot_idx, out)
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape or g.shape != k.shape or \
            (k.shape[0], k.shape[2], k.shape[3]) != (q.shape[0], q.shape[2], q.shape[3]):
        raise ValueError(f"q [B, H, T, D] and k, v, g [B, H or Hkv, T, D] expected; got {tuple(q.shape)}, "
                         f"{tuple(k.shape)}, {tuple(v.shape)}, {tuple(g.shape)}")
    B, H, T, D = q.shape
    Hk = _state_heads(H, k.shape[1])
    if not (k.dtype == q.dtype and v.dtype == q.dtype):
        raise ValueError("q, k, v must share one dtype")
    if state.dim() != 4 or state.shape[1:] != (Hk, D, D):
        raise ValueError(f"state must be [slots, {Hk}, {D}, {D}], got {tuple(state.shape)}")
    if state.stride(3) != 1 or state.stride(2) != D:
        raise ValueError("each [dk, dv] state matrix must be contiguous")
    for t, n in ((q, "q"), (k, "k"), (v, "v"), (g, "g")):
        _inner_contiguous(t, n)
    if slot_idx is not None:
        if slot_idx.dtype != torch.int32 or slot_idx.dim() != 1 or slot_idx.numel() < B or not slot_idx.is_contiguous():
            raise ValueError("slot_idx must be a contiguous int32 vector with one entry per batch row")
    elif state.shape[0] < B:
        raise ValueError(f"state has {state.shape[0]} slots for a batch of {B} and no slot_idx")
    if scale is None:
        scale = D ** -0.5
    if out is None:
        out = torch.empty((B, H, T, D), dtype=q.dtype, device=dev)
    else:
        if out.shape != q.shape or out.dtype != q.dtype:
            raise ValueError("out must match q in shape and dtype")
        _inner_contiguous(out, "out")
    a = N.GlaRecurrentArgs(
        q=N.ptr(q), k=N.ptr(k), v=N.ptr(v), g=N.ptr(g), state=N.ptr(state), out=N.ptr(out),
        slot_idx=N.ptr(slot_idx), batch=B, num_heads=H, seq_len=T, head_dim=D,
        dtype=N.dtype_code(q.dtype), g_dtype=N.dtype_code(g.dtype), state_dtype=N.dtype_code(state.dtype),
        scale=float(scale),
        q_stride_b=q.stride(0), q_stride_h=q.stride(1), q_stride_t=q.stride(2),
        k_stride_b=k.stride(0), k_stride_h=k.stride(1), k_stride_t=k.stride(2),
        v_stride_b=v.stride(0), v_stride_h=v.stride(1), v_stride_t=v.stride(2),
        g_stride_b=g.stride(0), g_stride_h=g.stride(1), g_stride_t=g.stride(2),
        out_stride_b=out.stride(0), out_stride_h=out.stride(1), out_stride_t=out.stride(2),
        state_stride_slot=state.stride(0), state_stride_head=state.stride(1),
        num_slots=state.shape[0], stream=N.stream_ptr(dev),
        flags=(N.SB_GLA_VECTOR_ONLY if vector_only else 0) | (N.SB_GLA_CHECK_GATES if check_gates else 0)
        | (0 if per_head is None else (N.SB_GLA_PER_HEAD if per_head else N.SB_GLA_GROUP_PASS)),
        q_heads_per_state=H // Hk, **_event_args(profile_events))
    N.check(N.lib().sb_gla_recurrent(C.byref(a)), "gla_recurrent")
    return out


def _state_heads(num_q_heads: int, num_k_heads: int) -> int:
    """Heads of k, v, g and of the state: all of them, or one per group of up to 8 query heads."""
    if num_k_heads <= 0 or num_q_heads % num_k_heads or num_q_heads // num_k_heads > 8:
        raise ValueError(f"{num_q_heads} query heads over {num_k_heads} heads of k, v, g: need a whole number of "
                         "query heads per head, at most 8")
    return num_k_heads


def gla_recurrent_packed(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
                         cu_seqlens: torch.Tensor, slot_idx: Optional[torch.Tensor] = None,
                         scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                         max_seq_len: Optional[int] = None, vector_only: bool = False,
                         check_gates: bool = False, per_head: Optional[bool] = None) -> torch.Tensor:
    """The same recurrence over packed prompts: q, k, v, g [total_tokens, H, D] (token/head strides
    free, contiguous D), sequence b owning tokens cu_seqlens[b] .. cu_seqlens[b+1]-1 (int32 device
    vector [B+1]); its state is state[slot_idx[b]] (default b), advanced in place. One launch for
    all sequences. Returns o [total_tokens, H, D]. Shared states as in gla_recurrent: k, v, g
    [total_tokens, Hkv, D] with state [slots, Hkv, D, D]."""
    dev = N.require_gpu(q, k, v, g, state, cu_seqlens, slot_idx, out)
    if q.dim() != 3 or k.dim() != 3 or v.shape != k.shape or g.shape != k.shape or \
            (k.shape[0], k.shape[2]) != (q.shape[0], q.shape[2]):
        raise ValueError("q [total_tokens, H, D] and k, v, g [total_tokens, H or Hkv, D] expected")
    Tt, H, D = q.shape
    Hk = _state_heads(H, k.shape[1])
    if not (k.dtype == q.dtype and v.dtype == q.dtype):
        raise ValueError("q, k, v must share one dtype")
    if state.dim() != 4 or state.shape[1:] != (Hk, D, D) or state.stride(3) != 1 or state.stride(2) != D:
        raise ValueError(f"state must be [slots, {Hk}, {D}, {D}] with contiguous matrices")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2 or not cu_seqlens.is_contiguous():
        raise ValueError("cu_seqlens must be a contiguous int32 vector [B+1]")
    B = cu_seqlens.numel() - 1
    for t, n in ((q, "q"), (k, "k"), (v, "v"), (g, "g")):
        _inner_contiguous(t, n)
    if slot_idx is not None:
        if slot_idx.dtype != torch.int32 or slot_idx.dim() != 1 or slot_idx.numel() < B or not slot_idx.is_contiguous():
            raise ValueError("slot_idx must be a contiguous int32 vector with one entry per sequence")
    elif state.shape[0] < B:
        raise ValueError(f"state has {state.shape[0]} slots for {B} sequences and no slot_idx")
    if scale is None:
        scale = D ** -0.5
    if out is None:
        out = torch.empty((Tt, H, D), dtype=q.dtype, device=dev)
    elif out.shape != q.shape or out.dtype != q.dtype or out.stride(-1) != 1:
        raise ValueError("out must match q in shape and dtype, with a contiguous last dimension")
    if Tt == 0:
        return out
    a = N.GlaRecurrentArgs(
        q=N.ptr(q), k=N.ptr(k), v=N.ptr(v), g=N.ptr(g), state=N.ptr(state), out=N.ptr(out),
        slot_idx=N.ptr(slot_idx), batch=B, num_heads=H, seq_len=int(max_seq_len or Tt), head_dim=D,
        dtype=N.dtype_code(q.dtype), g_dtype=N.dtype_code(g.dtype), state_dtype=N.dtype_code(state.dtype),
        scale=float(scale),
        q_stride_b=0, q_stride_h=q.stride(1), q_stride_t=q.stride(0),
        k_stride_b=0, k_stride_h=k.stride(1), k_stride_t=k.stride(0),
        v_stride_b=0, v_stride_h=v.stride(1), v_stride_t=v.stride(0),
        g_stride_b=0, g_stride_h=g.stride(1), g_stride_t=g.stride(0),
        out_stride_b=0, out_stride_h=out.stride(1), out_stride_t=out.stride(0),
        state_stride_slot=state.stride(0), state_stride_head=state.stride(1),
        num_slots=state.shape[0], stream=N.stream_ptr(dev), cu_seqlens=N.ptr(cu_seqlens),
        flags=(N.SB_GLA_VECTOR_ONLY if vector_only else 0) | (N.SB_GLA_CHECK_GATES if check_gates else 0)
        | (0 if per_head is None else (N.SB_GLA_PER_HEAD if per_head else N.SB_GLA_GROUP_PASS)),
        q_heads_per_state=H // Hk)
    N.check(N.lib().sb_gla_recurrent(C.byref(a)), "gla_recurrent")
    return out


def copy_blocks(cache_half: torch.Tensor, pairs: torch.Tensor) -> None:
    """cache_half [num_blocks, ...] with contiguous blocks; pairs [n, 2] int64 (src, dst) on the
    same device. One half (K or V) per call, as ops.copy_blocks does per layer at
    vllm_hymeta/attention/meta_attention.py:115-126."""
    dev = N.require_gpu(cache_half, pairs)
    if pairs.dtype != torch.int64 or pairs.dim() != 2 or pairs.shape[1] != 2:
        raise ValueError("pairs must be an int64 [n, 2] tensor")
    pairs = pairs.contiguous()
    if not cache_half[0].is_contiguous():
        raise ValueError("each cache block must be contiguous")
    esz = cache_half.element_size()
    N.check(N.lib().sb_copy_blocks(N.ptr(cache_half), N.ptr(pairs), pairs.shape[0],
                                   cache_half[0].numel() * esz, cache_half.stride(0) * esz,
                                   N.stream_ptr(dev)), "copy_blocks")


def stream_copy(dst: torch.Tensor, src: torch.Tensor) -> None:
    """Plain streaming device copy of contiguous tensors of equal byte size (a multiple of 16 KiB):
    the bandwidth yardstick of bench.py and the calibration launch for the HBM byte counters."""
    dev = N.require_gpu(dst, src)
    nbytes = src.numel() * src.element_size()
    if not (dst.is_contiguous() and src.is_contiguous()) or dst.numel() * dst.element_size() != nbytes:
        raise ValueError("stream_copy needs contiguous tensors of equal byte size")
    N.check(N.lib().sb_stream_copy(N.ptr(dst), N.ptr(src), nbytes, N.stream_ptr(dev)), "stream_copy")


def window_shift(src: Optional[torch.Tensor], dst: torch.Tensor, fresh: Optional[torch.Tensor], *, keep_rows: int,
                 src_row0: int, dst_row0: int) -> None:
    """dst[..., dst_row0 : dst_row0+keep_rows, :] = src[..., src_row0 : src_row0+keep_rows, :] and the
    n rows of fresh behind them; src/dst are [B, H, cap, D] contiguous, fresh is [B, H, n, D]."""
    dev = N.require_gpu(src, dst, fresh)
    B, H, cap_d, D = dst.shape
    if not dst.is_contiguous() or (src is not None and not src.is_contiguous()):
        raise ValueError("window_shift needs contiguous [B, H, cap, D] storage")
    esz = dst.element_size()
    n_new = 0 if fresh is None else fresh.shape[2]
    if fresh is not None:
        if fresh.shape[:2] != (B, H) or fresh.shape[3] != D or fresh.dtype != dst.dtype or fresh.stride(3) != 1:
            raise ValueError("fresh must be [B, H, n, D] of the cache dtype with contiguous rows")
        if fresh.stride(0) != H * fresh.stride(1):
            fresh = fresh.contiguous()
    if dst_row0 + keep_rows + n_new > cap_d:
        raise ValueError("window_shift would write past the destination capacity")
    a = N.WindowShiftArgs(
        src=N.ptr(src), dst=N.ptr(dst), fresh=N.ptr(fresh), planes=B * H, keep_rows=keep_rows,
        src_row0=src_row0, dst_row0=dst_row0, n_new=n_new, row_bytes=D * esz,
        src_stride_plane_bytes=0 if src is None else src.stride(1) * esz,
        dst_stride_plane_bytes=dst.stride(1) * esz,
        fresh_stride_plane_bytes=0 if fresh is None else fresh.stride(1) * esz,
        fresh_stride_row_bytes=0 if fresh is None else fresh.stride(2) * esz,
        stream=N.stream_ptr(dev))
    N.check(N.lib().sb_window_shift(C.byref(a)), "window_shift")


def window_advance(n_tokens: torch.Tensor, lo: torch.Tensor, hi: torch.Tensor, ring: torch.Tensor,
                   free_stack: torch.Tensor, free_top: torch.Tensor, slot_mapping: torch.Tensor,
                   seq_lens: torch.Tensor, block_tables: torch.Tensor, status: torch.Tensor, *,
                   block_size: int, window_left: int) -> None:
    """One decode token for every sequence, on the device: evict / allocate / slot / visible length /
    block-table rows, with the host block manager's policy (see block_manager.DeviceWindowState).
    All tensors are updated in place; nothing is allocated and nothing is read back."""
    dev = N.require_gpu(n_tokens, lo, hi, ring, free_stack, free_top, slot_mapping, seq_lens, block_tables, status)
    B = n_tokens.numel()
    want = ((n_tokens, torch.int64, (B,)), (lo, torch.int32, (B,)), (hi, torch.int32, (B,)),
            (free_top, torch.int32, (1,)), (slot_mapping, torch.int64, (B,)), (seq_lens, torch.int32, (B,)),
            (status, torch.int32, (1,)))
    for t, dt, shape in want:
        if t.dtype != dt or tuple(t.shape) != shape or not t.is_contiguous():
            raise ValueError(f"window_advance: expected a contiguous {dt} tensor of shape {shape}, got "
                             f"{t.dtype} {tuple(t.shape)}")
    for t, name in ((ring, "ring"), (block_tables, "block_tables")):
        if t.dtype != torch.int32 or t.dim() != 2 or t.shape[0] != B or not t.is_contiguous():
            raise ValueError(f"window_advance: {name} must be a contiguous int32 [batch, n] tensor")
    if free_stack.dtype != torch.int32 or free_stack.dim() != 1 or not free_stack.is_contiguous():
        raise ValueError("window_advance: free_stack must be a contiguous int32 vector")
    a = N.WindowAdvanceArgs(
        n_tokens=N.ptr(n_tokens), lo=N.ptr(lo), hi=N.ptr(hi), ring=N.ptr(ring), free_stack=N.ptr(free_stack),
        free_top=N.ptr(free_top), slot_mapping=N.ptr(slot_mapping), seq_lens=N.ptr(seq_lens),
        block_tables=N.ptr(block_tables), status=N.ptr(status), batch=B, ring_blocks=ring.shape[1],
        block_size=int(block_size), window_left=int(window_left), table_width=block_tables.shape[1],
        num_blocks=free_stack.numel(), stream=N.stream_ptr(dev))
    N.check(N.lib().sb_window_advance(C.byref(a)), "window_advance")
