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


# ---- fp8 (OCP e4m3fn) with per-tensor scales ---------------------------------------------------------
# The kv_cache_dtype="fp8" branch of reshape_and_cache_flash (vllm_hymeta/attention/meta_attention.py:790-799)
# and scaled_fp8_quant (:806-811, :853-869). The kernels live in vllm 0.10.0, absent here: restated from
# its published behaviour, code = e4m3fn(x / scale) with saturation at +-448 and round to nearest even.
# The rounding itself is torch's own float8_e4m3fn cast (a library routine, checked code by code in
# tests/test_oracle_quant.py); parity with vllm's kernel is unpinned.

def fp8_codes(x: np.ndarray, scale: float) -> np.ndarray:
    """uint8 e4m3fn codes of x / scale (float32 division, saturating, ties to even, NaN kept)."""
    import torch
    y = torch.from_numpy(np.ascontiguousarray(x, np.float32)) / np.float32(scale)
    y = torch.where(torch.isnan(y), y, y.clamp(-448.0, 448.0))
    return y.to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def fp8_values(codes: np.ndarray, scale: float) -> np.ndarray:
    """float32 value of each code times scale."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(codes, np.uint8)).view(torch.float8_e4m3fn).float().numpy() * np.float32(scale)


def fp8_round(x: np.ndarray, scale: float, dtype: str = "bf16") -> np.ndarray:
    """x after the fp8 round trip, rounded to the tensor's dtype; returned as float32."""
    y = fp8_values(fp8_codes(x, scale), scale)
    if dtype == "bf16":
        return round_to_bf16(y)
    if dtype == "f16":
        return y.astype(np.float16).astype(np.float32)
    return y
