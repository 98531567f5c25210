"""numpy restatement of the per-row symmetric INT8 quantisation of cached K/V.

TEST INFRASTRUCTURE: see oracle/__init__.py.

Follows quantize_sym, W8ASpike/window_attention.py:227-237, as applied to key_states and
value_states at :183-186: per row of the last axis, in float32,
  scale = clamp(max|x| / 127, 1e-5, 1e4); code = clamp(round(x / scale), -128, 127)   (round half to even)
and the value attention sees is code * scale rounded to the tensor's dtype.
"""
from __future__ import annotations

from typing import Sequence, Tuple

import numpy as np


def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(x))


def quantize_rows(x: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """(codes int8 [..., D], scale float32 [...]) of quantize_sym (:228-234), float32 arithmetic."""
    x = np.asarray(x, np.float32)
    scale = np.abs(x).max(-1).astype(np.float32) / np.float32(127)
    scale = np.clip(scale, np.float32(1e-5), np.float32(1e4)).astype(np.float32)
    codes = np.clip(np.rint(x / scale[..., None]), -128, 127)
    return codes.astype(np.int8), scale


def dequantize_rows(codes: np.ndarray, scale: np.ndarray, dtype: str = "bf16") -> np.ndarray:
    """code * scale in float32, rounded to the tensor's dtype (:235-237); returned as float32."""
    y = codes.astype(np.float32) * np.asarray(scale, np.float32)[..., None]
    if dtype == "bf16":
        return round_to_bf16(y)
    if dtype == "f16":
        with np.errstate(over="ignore"):     # beyond 65504 the half-precision value is inf, as in torch
            return y.astype(np.float16).astype(np.float32)
    return y


def quantize_sym(x: np.ndarray, dtype: str = "bf16") -> np.ndarray:
    codes, scale = quantize_rows(x)
    return dequantize_rows(codes, scale, dtype)


def kv_append_int8(key: np.ndarray, value: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
                   k_scale: np.ndarray, v_scale: np.ndarray, slot_mapping: Sequence[int]) -> None:
    """Slot-mapped append (the contract of reshape_and_cache_flash,
    vllm_hymeta/attention/meta_attention.py:790-799) into int8 caches [nb, bs, Hkv, D] with scales
    [nb, Hkv, bs]; slots < 0 are skipped."""
    bs = k_cache.shape[1]
    kc, ks = quantize_rows(key)
    vc, vs = quantize_rows(value)
    for t, slot in enumerate(slot_mapping):
        if slot < 0:
            continue
        b, o = divmod(int(slot), bs)
        k_cache[b, o] = kc[t]; v_cache[b, o] = vc[t]
        k_scale[b, :, o] = ks[t]; v_scale[b, :, o] = vs[t]
