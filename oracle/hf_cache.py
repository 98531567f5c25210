"""numpy restatement of hf_7B_model/cache.py (the HuggingFace-side per-layer state store).

TEST INFRASTRUCTURE: see oracle/__init__.py.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import numpy as np


class OracleCache:
    """Follows hf_7B_model/cache.py:11-139 statement by statement on numpy arrays.

    attn_state tensors are [B, Hkv, L, D]; all operations are copies, so results are
    bit-exact restatements (roll -> np.roll, cat -> np.concatenate).
    """

    def __init__(self, seen_tokens: int = 0):
        # cache.py:19-25
        self.states: List[Dict[str, Any]] = []
        self._seen_tokens = seen_tokens

    def __getitem__(self, layer_idx: int):
        # cache.py:27-31
        if layer_idx < len(self):
            return self.states[layer_idx]
        raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")

    def __iter__(self):
        yield from self.states

    def __len__(self):
        return len(self.states)

    def update(self, recurrent_state=None, attn_state=None, conv_state=None, layer_idx: int = 0,
               offset: Optional[int] = 1, cache_kwargs: Optional[Dict[str, Any]] = None) -> Dict[str, Any]:
        # cache.py:69-71 — only layer 0 advances the token counter
        if layer_idx == 0:
            self._seen_tokens += offset
        if attn_state is not None:
            # cache.py:73-78 — note: indexing happens before the tuple check, as in the reference
            input_size = attn_state[0].shape[-2]
            window_size = cache_kwargs.get("window_size", None)
            if not isinstance(attn_state, tuple) or len(attn_state) != 2:
                raise ValueError("`attn_state` must be a tuple of two tensors for key/value states")
        if len(self.states) <= layer_idx:
            # cache.py:79-89 — first call for this layer: truncate to the last window_size rows
            if attn_state is not None:
                if window_size is not None and input_size > window_size:
                    attn_state = (np.ascontiguousarray(attn_state[0][..., -window_size:, :]),
                                  np.ascontiguousarray(attn_state[1][..., -window_size:, :]))
            state = dict(recurrent_state=recurrent_state, attn_state=attn_state, conv_state=conv_state)
            self.states.append(state)
        else:
            state = self.states[layer_idx]
            if recurrent_state is not None:
                state["recurrent_state"] = recurrent_state  # cache.py:92-93 (by reference)
            if attn_state is not None:
                key_state, value_state = state["attn_state"]
                if window_size is not None and key_state.shape[-2] == window_size:
                    # cache.py:96-104 — equality test, roll left, overwrite the tail
                    key_state = np.roll(key_state, -input_size, axis=-2)
                    value_state = np.roll(value_state, -input_size, axis=-2)
                    key_state[..., -input_size:, :] = attn_state[0]
                    value_state[..., -input_size:, :] = attn_state[1]
                    attn_state = (key_state, value_state)
                else:
                    # cache.py:105-107
                    attn_state = (np.concatenate([key_state, attn_state[0]], -2),
                                  np.concatenate([value_state, attn_state[1]], -2))
                state["attn_state"] = attn_state
            if conv_state is not None:
                state["conv_state"] = conv_state  # cache.py:109-110
        return state

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        # cache.py:114-118 — the global counter, not the cached length
        if len(self.states) <= layer_idx:
            return 0
        return self._seen_tokens

    def get_max_length(self) -> Optional[int]:
        return None  # cache.py:120-122

    def to_legacy_cache(self) -> Tuple[Dict[str, Any], ...]:
        return tuple(self.states)  # cache.py:124-125

    @classmethod
    def from_legacy_cache(cls, past_key_values=None, seen_tokens: int = 0) -> "OracleCache":
        # cache.py:127-139
        cache = cls(seen_tokens)
        if past_key_values is not None:
            for layer_idx in range(len(past_key_values)):
                cache.states.append(past_key_values[layer_idx])
        return cache
