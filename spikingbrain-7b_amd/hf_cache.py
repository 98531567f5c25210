"""HuggingFace-side per-layer state store: drop-in for hf_7B_model/cache.py.

Same class name, method names, argument meaning, return values and exceptions as the reference
`Cache` (cache.py:11-139). What differs is how the sliding-window K/V are kept in GPU memory:

  reference   every decode token `roll`s and rewrites the whole [B, Hkv, W, D] pair
              (cache.py:96-104): O(W) bytes moved per token per layer;
  here        each K/V lives in a [B, Hkv, capacity, D] buffer with capacity > W and the
              cache is the row window [start, start+L) of it. A token is written behind the
              window by a HIP copy kernel and the window slides by moving `start`; only when
              the window reaches the end of the buffer is it copied back to the front (once
              every capacity-W tokens), so the amortised traffic is O(1) rows per token.

The tensors handed back in `state['attn_state']` are strided views [B, Hkv, L, D] of those
buffers: chronological, bit-identical in content to what the reference would hold, but they
alias the buffers, so a view is valid until the next `update` of that layer (the reference's
callers, window_attention.py:166-177, consume it immediately).
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from . import ops


class _WindowBuffer:
    """K or V rows of one layer: storage [B, H, cap, D], live rows [start, start+length)."""

    __slots__ = ("storage", "start", "length")

    def __init__(self, storage: torch.Tensor, start: int, length: int):
        self.storage = storage
        self.start = start
        self.length = length

    def view(self) -> torch.Tensor:
        return self.storage[:, :, self.start:self.start + self.length, :]


def _capacity_for(rows: int, window: Optional[int]) -> int:
    # room for the window plus as many appended tokens again before a compaction is due
    base = max(rows, window or 0)
    return ((2 * base + 64 + 15) // 16) * 16


try:  # the reference's class derives from transformers' Cache (cache.py:9-11); so does this one when it is there
    from transformers.cache_utils import Cache as _HFCache
except Exception:  # transformers missing or too old to have cache_utils
    _HFCache = object


class Cache(_HFCache):
    """Drop-in for the reference `Cache` (hf_7B_model/cache.py:11).

    states[layer] is a dict with keys recurrent_state / attn_state / conv_state, appended in
    layer order on each layer's first `update`. Like the reference it subclasses
    `transformers.cache_utils.Cache` without calling its constructor (cache.py:19-25), so callers
    that test `isinstance(past_key_values, transformers.Cache)` (HF generate plumbing) accept it;
    every method those callers use is overridden here, none of the base class's own storage exists
    (`layers` is an empty list).
    """

    def __init__(self, seen_tokens: int = 0):
        self.layers = []  # the transformers base class's own per-layer storage: unused, kept empty
        self.states: List[Dict[str, Any]] = []
        self._seen_tokens = seen_tokens  # cache.py:25
        self._buffers: Dict[int, Tuple[_WindowBuffer, _WindowBuffer]] = {}

    def __getitem__(self, layer_idx: int) -> Dict[str, Any]:
        if layer_idx < len(self):
            return self.states[layer_idx]
        raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")

    def __iter__(self):
        for state in self.states:
            yield state

    def __len__(self):
        return len(self.states)

    # -- sliding-window storage ---------------------------------------------------------
    @staticmethod
    def _new_buffer(rows: torch.Tensor, window: Optional[int]) -> _WindowBuffer:
        """Store `rows` [B, H, n, D] (already truncated) in a fresh buffer."""
        B, H, n, D = rows.shape
        storage = torch.empty((B, H, _capacity_for(n, window), D), dtype=rows.dtype, device=rows.device)
        ops.window_shift(None, storage, rows, keep_rows=0, src_row0=0, dst_row0=0)
        return _WindowBuffer(storage, 0, n)

    @staticmethod
    def _push(buf: _WindowBuffer, rows: torch.Tensor, drop: int, window: Optional[int]) -> None:
        """Drop the `drop` oldest live rows and append `rows` behind the rest."""
        n = rows.shape[2]
        keep = buf.length - drop
        cap = buf.storage.shape[2]
        if buf.start + buf.length + n <= cap:
            ops.window_shift(None, buf.storage, rows, keep_rows=0, src_row0=0, dst_row0=buf.start + buf.length)
            buf.start += drop
        elif keep + n <= buf.start + drop:
            # compaction: kept rows move to the front of the same buffer; every destination row
            # (kept + new) lies below the first source row, so the copy cannot race with itself
            ops.window_shift(buf.storage, buf.storage, rows, keep_rows=keep, src_row0=buf.start + drop, dst_row0=0)
            buf.start = 0
        else:
            B, H, _, D = buf.storage.shape
            storage = torch.empty((B, H, _capacity_for(keep + n, window), D), dtype=rows.dtype, device=rows.device)
            ops.window_shift(buf.storage, storage, rows, keep_rows=keep, src_row0=buf.start + drop, dst_row0=0)
            buf.storage = storage
            buf.start = 0
        buf.length = keep + n

    def update(
        self,
        recurrent_state: torch.Tensor = None,
        attn_state: Tuple[torch.Tensor, torch.Tensor] = None,
        conv_state: Tuple[torch.Tensor] = None,
        layer_idx: int = 0,
        offset: Optional[int] = 1,
        cache_kwargs: Optional[Dict[str, Any]] = None,
    ) -> Dict[str, Any]:
        """Same contract as cache.py:40-112. `attn_state` = (key, value), each [B, Hkv, n, D];
        `cache_kwargs['window_size']` bounds the stored rows (None = unbounded)."""
        if layer_idx == 0:
            self._seen_tokens += offset  # cache.py:70-71: only layer 0 counts tokens

        if attn_state is not None:
            input_size = attn_state[0].shape[-2]
            window_size = cache_kwargs.get("window_size", None)
            if not isinstance(attn_state, tuple) or len(attn_state) != 2:
                raise ValueError("`attn_state` must be a tuple of two tensors for key/value states")
        if len(self.states) <= layer_idx:
            if attn_state is not None:
                k_new, v_new = attn_state
                if window_size is not None and input_size > window_size:
                    k_new = k_new[..., -window_size:, :]
                    v_new = v_new[..., -window_size:, :]
                kb = self._new_buffer(k_new, window_size)
                vb = self._new_buffer(v_new, window_size)
                self._buffers[len(self.states)] = (kb, vb)
                attn_state = (kb.view(), vb.view())
            state = dict(recurrent_state=recurrent_state, attn_state=attn_state, conv_state=conv_state)
            self.states.append(state)
        else:
            state = self.states[layer_idx]
            if recurrent_state is not None:
                state["recurrent_state"] = recurrent_state
            if attn_state is not None:
                bufs = self._buffers.get(layer_idx)
                if bufs is None:  # layer entry came from from_legacy_cache or held no K/V yet
                    old = state["attn_state"]
                    if old is None:
                        raise TypeError("'NoneType' object is not iterable")  # what unpacking None raises
                    bufs = (self._new_buffer(old[0], window_size), self._new_buffer(old[1], window_size))
                    self._buffers[layer_idx] = bufs
                kb, vb = bufs
                # cache.py:96: the window slides only when the stored length EQUALS the window;
                # otherwise rows are concatenated (so an overshoot is never trimmed)
                drop = input_size if (window_size is not None and kb.length == window_size) else 0
                if drop > kb.length:
                    raise RuntimeError(
                        f"cannot roll {input_size} new rows into a window of {kb.length}: the reference's "
                        "slice-assign would fail with a shape mismatch here")
                self._push(kb, attn_state[0], drop, window_size)
                self._push(vb, attn_state[1], drop, window_size)
                state["attn_state"] = (kb.view(), vb.view())
            if conv_state is not None:
                state["conv_state"] = conv_state
        return state

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        """cache.py:114-118: 0 until the layer has an entry, then the global token counter."""
        if len(self.states) <= layer_idx:
            return 0
        return self._seen_tokens

    def get_max_length(self) -> Optional[int]:
        return None

    def to_legacy_cache(self) -> Tuple[Dict[str, Any], ...]:
        return tuple(self.states)

    @classmethod
    def from_legacy_cache(cls, past_key_values: Optional[Tuple[Dict[str, Any], ...]] = None,
                          seen_tokens: int = 0) -> "Cache":
        """cache.py:127-139. Layer dicts are adopted as they are; a layer whose K/V came in this way
        is re-homed into a window buffer on its next `update`."""
        cache = cls(seen_tokens)
        if past_key_values is not None:
            for layer_idx in range(len(past_key_values)):
                cache.states.append(past_key_values[layer_idx])
        return cache

    # -- extension used by the attention slice: where a layer's K/V live ------------------
    def dense_layout(self, layer_idx: int):
        """(key_view, value_view, row capacity) of a layer, or None if it has no window buffer."""
        bufs = self._buffers.get(layer_idx)
        if bufs is None:
            return None
        return bufs[0].view(), bufs[1].view(), bufs[0].storage.shape[2]
