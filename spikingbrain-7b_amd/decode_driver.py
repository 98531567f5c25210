"""Cache side of the hybrid stack's decode loop: what the reference's model forward does to the
caches on every generated token, with the projections, norms and MLPs left to the caller.

Layer order follows hf_7B_model/configuration_gla_swa.py:75 (even layers GLA, odd layers sliding
window). Per step and sequence
  * every GLA layer reads and rewrites its [H, D, D] fp32 state at the sequence's slot
    (vllm_hymeta/model_for_7B/gla_attention.py:223-235 -> my_fused_recurrent_gla);
  * every SWA layer appends the new K/V row at the step's slot and attends inside the window
    (vllm_hymeta/attention/meta_attention.py:767-799, 920-981), all SWA layers sharing ONE block table
    and slot mapping (each layer has its own KV tensor indexed by the same block ids);
  * the block manager evicts the block that left the window and hands its id to the block the
    sequence grows into (one recycle per sequence every block_size steps once the window is full).

The step metadata comes from the block manager's vectorised host path (numpy over the batch; only
sequences that cross a block boundary do per-sequence work) and three small uploads.
"""
from __future__ import annotations

from typing import List, Optional

import numpy as np
import torch

from . import ops
from .block_manager import DeviceWindowState, WindowBlockManager
from .meta_attention import MetaAttentionBackend, MetaAttentionImpl, MetaAttentionMetadata


class HybridDecodeCache:
    def __init__(self, batch: int, *, num_layers: int = 28, num_heads: int = 28, num_kv_heads: int = 4,
                 head_size: int = 128, block_size: int = 16, window_left: int = 4096,
                 dtype: torch.dtype = torch.bfloat16, device="cuda:0", num_blocks: Optional[int] = None,
                 randomize: bool = False, seed: int = 0, kv_quant: Optional[str] = None,
                 gla_state_dtype: torch.dtype = torch.float32, gla_shared_states: bool = False):
        """kv_quant="int8": the SWA layers keep their K/V as per-row INT8 codes + fp32 scales
        (quantize_sym of W8ASpike/window_attention.py:227-237 applied once, at append time);
        kv_quant="fp8": as e4m3fn codes with per-tensor scales of 1 (the kv_cache_dtype="fp8" branch of
        vllm_hymeta/attention/meta_attention.py:790-812).
        gla_state_dtype: float32, or bfloat16 as the reference's serving path keeps its state cache
        (vllm_hymeta/model_for_7B/modeling_gla_swa.py:361-364); the arithmetic is fp32 either way.
        gla_shared_states: keep one GLA state per kv head instead of one per query head; the layers then
        take k, v, g with num_kv_heads heads, before the model's repeat_kv
        (vllm_hymeta/model_for_7B/gla_attention.py:264-267), and give the same outputs."""
        if gla_state_dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("gla_state_dtype must be float32 or bfloat16")
        if kv_quant not in (None, "int8", "fp8"):
            raise ValueError(f"kv_quant {kv_quant!r} (None, 'int8' or 'fp8')")
        self.kv_quant = kv_quant
        self.device = torch.device(device)
        self.batch, self.num_layers = batch, num_layers
        self.H, self.Hkv, self.D, self.bs, self.wl = num_heads, num_kv_heads, head_size, block_size, window_left
        self.swa_layers = [i for i in range(num_layers) if i % 2 == 1]
        self.gla_layers = [i for i in range(num_layers) if i % 2 == 0]
        per_seq = (window_left + 1) // block_size + 2
        self.num_blocks = num_blocks if num_blocks is not None else batch * per_seq + 8
        self.manager = WindowBlockManager(self.num_blocks, block_size, window_left, batch)
        shape = MetaAttentionBackend.get_kv_cache_shape(self.num_blocks, block_size, num_kv_heads, head_size)
        g = torch.Generator(device=self.device).manual_seed(seed)

        def alloc(shape, dt, std):
            if randomize:
                return torch.randn(shape, dtype=torch.float32, device=self.device, generator=g).mul_(std).to(dt) \
                    if dt != torch.float32 else torch.randn(shape, dtype=dt, device=self.device, generator=g).mul_(std)
            return torch.zeros(shape, dtype=dt, device=self.device)

        if kv_quant == "int8":
            self.kv_caches, self.kv_scales = [], []
            for _ in self.swa_layers:
                codes, scales = ops.alloc_int8_kv_cache(self.num_blocks, block_size, num_kv_heads, head_size, self.device)
                if randomize:
                    codes.random_(-127, 128, generator=g)
                    scales.uniform_(0.005, 0.03, generator=g)
                self.kv_caches.append(codes)
                self.kv_scales.append(scales)
        elif kv_quant == "fp8":
            self.kv_caches = []
            for _ in self.swa_layers:
                codes = torch.zeros(shape, dtype=torch.uint8, device=self.device)
                if randomize:   # finite codes only: 0x7f / 0xff are NaN
                    codes.random_(0, 0x7F, generator=g)
                self.kv_caches.append(codes)
        else:
            self.kv_caches: List[torch.Tensor] = [alloc(shape, dtype, 1.0) for _ in self.swa_layers]
        # [n_gla_layers, slots, H, D, D] fp32, as vllm_hymeta/model_for_7B/modeling_gla_swa.py:348-356
        self.gla_state_heads = num_kv_heads if gla_shared_states else num_heads
        self.gla_state = alloc((len(self.gla_layers), batch, self.gla_state_heads, head_size, head_size),
                               gla_state_dtype, 0.02)
        self.slot_idx = torch.arange(batch, dtype=torch.int32, device=self.device)
        self.impl = MetaAttentionImpl(num_heads, head_size, head_size ** -0.5, num_kv_heads, None, window_left + 1,
                                      "auto")
        self.seq_ids = list(range(batch))
        for s in self.seq_ids:
            self.manager.add_seq(s)
        self._gla_out = torch.empty(batch, num_heads, 1, head_size, dtype=dtype, device=self.device)
        self._layer = _Layer()

    def start(self, context_len: int) -> None:
        """Every sequence already holds `context_len` tokens: only the blocks inside the window get
        ids (what a prompt run leaves behind); the cache contents are whatever the tensors hold."""
        for s in self.seq_ids:
            self.manager.append_tokens(s, context_len, True)

    _STAGES = 4   # staging sets: the host may run this many steps ahead of the GPU

    def _staging(self):
        """A ring of `_STAGES` staging sets, each a pair of pinned host buffers (the step's slots | lengths and
        its block tables are written there, so that their uploads are truly asynchronous: from pageable
        memory a `non_blocking` copy still waits for the stream, which lock-steps the host to the GPU) and
        the device tensors they are uploaded into. The uploads run on a stream of their own, beside the
        layers of the step before; the layers' stream waits for them. A set is rewritten only after the
        layers of the step that used it have run (an event recorded behind them when the next step's
        metadata is asked for), so the host runs at most `_STAGES` steps ahead."""
        if not hasattr(self, "_stage_sets"):
            B, width, dev = self.batch, self.manager.ring_blocks, self.device
            self._stage_sets = [dict(packed=torch.empty(2 * B, dtype=torch.int64).pin_memory(),
                                     tables=torch.empty(B * width, dtype=torch.int32).pin_memory(),
                                     d_packed=torch.empty(2 * B, dtype=torch.int64, device=dev),
                                     d_tables=torch.empty(B * width, dtype=torch.int32, device=dev),
                                     uploaded=torch.cuda.Event(), used=None) for _ in range(self._STAGES)]
            self._stage_next = 0
            self._stage_last = None
            self._upload_stream = torch.cuda.Stream(device=dev)
            self.host_wait_s = 0.0   # time spent waiting for a staging set (the GPU is that far behind)
        cur = torch.cuda.current_stream(self.device)
        if self._stage_last is not None:   # the layers of the previous step are all enqueued by now
            last = self._stage_sets[self._stage_last]
            if last["used"] is None:
                last["used"] = torch.cuda.Event()
            last["used"].record(cur)
        st = self._stage_sets[self._stage_next]
        self._stage_last = self._stage_next
        self._stage_next = (self._stage_next + 1) % self._STAGES
        if st["used"] is not None and not st["used"].query():
            import time
            t0 = time.perf_counter()
            st["used"].synchronize()
            self.host_wait_s += time.perf_counter() - t0
        return st

    def step_metadata(self) -> MetaAttentionMetadata:
        """Advance every sequence by one token (eviction + allocation) and build the decode-only
        metadata the SWA layers of this step share."""
        mgr = self.manager
        slots = mgr.decode_step(self.seq_ids)
        tables, seqlens, _ = mgr.kernel_view(self.seq_ids)
        dev = self.device
        B, width = self.batch, tables.shape[1]
        st = self._staging()
        hp = st["packed"].numpy()
        hp[:B] = slots
        hp[B:] = seqlens
        st["tables"][:B * width].view(B, width).numpy()[...] = tables
        with torch.cuda.stream(self._upload_stream):
            st["d_packed"].copy_(st["packed"], non_blocking=True)
            st["d_tables"][:B * width].copy_(st["tables"][:B * width], non_blocking=True)
            st["uploaded"].record(self._upload_stream)
        torch.cuda.current_stream(dev).wait_event(st["uploaded"])
        packed = st["d_packed"]
        return MetaAttentionMetadata(
            num_prefills=0, num_prefill_tokens=0, num_decode_tokens=B,
            slot_mapping=packed[:B], seq_lens=None, seq_lens_tensor=packed[B:].to(torch.int32),
            max_prefill_seq_len=0, max_decode_seq_len=int(seqlens.max()), context_lens_tensor=None,
            block_tables=st["d_tables"][:B * width].view(B, width), use_cuda_graph=False,
            max_query_len=1, max_decode_query_len=1)

    # -- device-side stepping: no host work between decode steps --------------------------------
    def enable_device_advance(self) -> MetaAttentionMetadata:
        """Move the block manager's state for this batch to the GPU. Returns the metadata object of
        every following step: its slot_mapping / seq_lens / block_tables are the tensors the advance
        kernels rewrite in place (`advance_device`), so one object (and one captured graph) serves
        all steps."""
        self.device_state = DeviceWindowState(self.manager, self.seq_ids, self.device)
        st = self.device_state
        B = self.batch
        self.device_meta = MetaAttentionMetadata(
            num_prefills=0, num_prefill_tokens=0, num_decode_tokens=B,
            slot_mapping=st.slot_mapping, seq_lens=None, seq_lens_tensor=st.seq_lens,
            max_prefill_seq_len=0, max_decode_seq_len=st.table_width * self.bs, context_lens_tensor=None,
            block_tables=st.block_tables, use_cuda_graph=True, max_query_len=1, max_decode_query_len=1)
        return self.device_meta

    def advance_device(self) -> None:
        """Enqueue the step advance (eviction, allocation, slots, lengths, tables) on the GPU."""
        self.device_state.advance()

    def capture_step(self, run_layers) -> "torch.cuda.CUDAGraph":
        """Capture `advance_device()` followed by `run_layers(meta)` (the caller's 28 layer calls on
        static input tensors) into one graph; every replay is one whole decode step."""
        meta = self.device_meta
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):      # warm up outside the capture: lazy allocations happen here
            self.advance_device()
            run_layers(meta)
        torch.cuda.current_stream(self.device).wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        before = set(ops.graph_workspace_ids(self.device))
        with torch.cuda.graph(graph):
            self.advance_device()
            run_layers(meta)
        # split-K workspaces this capture allocated belong to the graph: `release_step_graph` frees them
        graph.sb_workspace_ids = [c for c in ops.graph_workspace_ids(self.device) if c not in before]
        return graph

    def release_step_graph(self, graph) -> int:
        """Call when a graph from `capture_step` is dropped (re-capture for another batch size): hands the
        split-K workspaces it owned back to the allocator. The graph must not be replayed afterwards."""
        freed = 0
        for cid in getattr(graph, "sb_workspace_ids", []):
            freed += ops.release_graph_workspace(cid, self.device)
        graph.sb_workspace_ids = []
        return freed

    def gla_layer(self, layer_idx: int, q, k, v, g, out=None) -> torch.Tensor:
        """q [B, H, 1, D]; k, v, g [B, H, 1, D], or [B, Hkv, 1, D] with shared states; the layer's state is
        advanced in place. Returns o [B, H, 1, D]."""
        out = self._gla_out if out is None else out
        ops.gla_recurrent(q, k, v, g, self.gla_state[layer_idx // 2], self.slot_idx, self.D ** -0.5, out)
        return out

    def swa_layer(self, layer_idx: int, q, k, v, meta: MetaAttentionMetadata, out) -> torch.Tensor:
        """q [B, Hq, D], k/v [B, Hkv, D]: append + window attention for one SWA layer."""
        if self.kv_quant == "int8":
            codes, scales = self.kv_caches[layer_idx // 2], self.kv_scales[layer_idx // 2]
            n = q.shape[0]
            ops.kv_append_int8(k, v, codes[0], codes[1], scales[0], scales[1], meta.slot_mapping.flatten()[:n])
            return ops.swa_decode_attention(
                q, codes[0], codes[1], meta.seq_lens_tensor[:n], block_table=meta.block_tables, window_left=self.wl,
                scale=self.D ** -0.5, out=out, max_seq_len=meta.max_decode_seq_len or None,
                k_scale=scales[0], v_scale=scales[1])
        if self.kv_quant == "fp8":
            codes = self.kv_caches[layer_idx // 2]
            n = q.shape[0]
            ops.kv_append_fp8(k, v, codes[0], codes[1], meta.slot_mapping.flatten()[:n], 1.0, 1.0)
            return ops.swa_decode_attention(
                q, codes[0], codes[1], meta.seq_lens_tensor[:n], block_table=meta.block_tables, window_left=self.wl,
                scale=self.D ** -0.5, out=out, max_seq_len=meta.max_decode_seq_len or None, fp8_scales=(1.0, 1.0))
        return self.impl.forward(self._layer, q, k, v, None, None, None, self.kv_caches[layer_idx // 2], meta, out)

    def bytes_per_step(self) -> int:
        """Algorithmic HBM bytes of one decode step over all layers (window-saturated sequences)."""
        e = self._gla_out.element_size()
        n_keys = np.minimum(self.manager.n_tokens[:self.batch], self.wl + 1)
        if self.kv_quant == "fp8":      # per key and kv head: 2 x 128 code bytes
            swa = int(n_keys.sum()) * self.Hkv * 2 * self.D + self.batch * (
                2 * self.H * self.D * e + 2 * self.Hkv * self.D * e + self.Hkv * 2 * self.D)
        elif self.kv_quant == "int8":   # per key and kv head: 2 x 128 code bytes + 2 fp32 scales; new row read in e, written as codes
            swa = int(n_keys.sum()) * self.Hkv * (2 * self.D + 8) + self.batch * (
                2 * self.H * self.D * e + 2 * self.Hkv * self.D * e + self.Hkv * (2 * self.D + 8))
        else:
            swa = int(n_keys.sum()) * self.Hkv * self.D * 2 * e + self.batch * (2 * self.H * self.D * e
                                                                               + 4 * self.Hkv * self.D * e)
        # per state: read + write, and its k, v (e bytes) and gate (fp32) rows; per query head: q in, o out
        Hs = self.gla_state_heads
        gla = self.batch * (Hs * (2 * self.D * self.D * self.gla_state.element_size() + 2 * self.D * e + self.D * 4)
                            + self.H * 2 * self.D * e)
        return len(self.swa_layers) * swa + len(self.gla_layers) * gla


class _Layer:
    _k_scale_float = 1.0
    _v_scale_float = 1.0
