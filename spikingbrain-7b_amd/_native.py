"""ctypes binding of libsbcache.so (the C ABI declared in include/sbcache.h).

The library is the only compute path: there is no Python or CPU fallback. Loading fails loudly
when the shared object is missing, and every wrapper raises when a launch is rejected.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch  # imported first on purpose: the library must bind to the HIP runtime torch loaded

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsbcache.so")

SB_BF16, SB_F16, SB_F32 = 0, 1, 2
SB_ERR_INVALID, SB_ERR_UNSUPPORTED, SB_ERR_WORKSPACE = -1, -2, -3
SB_DECODE_FORCE_VALU = 1
SB_DECODE_BALANCED = 2
SB_DECODE_MERGE_IN_KERNEL = 4
SB_DECODE_PER_SEGMENT = 8
SB_KV_NONE, SB_KV_INT8, SB_KV_FP8 = 0, 1, 2
SB_GLA_VECTOR_ONLY = 1
SB_GLA_CHECK_GATES = 2
SB_GLA_PER_HEAD = 4
SB_GLA_GROUP_PASS = 8
SB_SWA_DECODE_STATIC_SCRATCH_BYTES = 8 << 20
ABI_VERSION = 3

_DTYPES = {torch.bfloat16: SB_BF16, torch.float16: SB_F16, torch.float32: SB_F32}

i32, i64, f32, vp, sz = C.c_int32, C.c_int64, C.c_float, C.c_void_p, C.c_size_t


class KvAppendArgs(C.Structure):
    _fields_ = [
        ("key", vp), ("value", vp), ("k_cache", vp), ("v_cache", vp), ("slot_mapping", vp),
        ("num_tokens", i64), ("num_kv_heads", i32), ("head_size", i32), ("block_size", i32),
        ("dtype", i32),
        ("key_stride_token", i64), ("key_stride_head", i64),
        ("value_stride_token", i64), ("value_stride_head", i64),
        ("cache_stride_block", i64), ("cache_stride_row", i64), ("cache_stride_head", i64),
        ("num_blocks", i64), ("stream", vp),
    ]


class SwaDecodeArgs(C.Structure):
    _fields_ = [
        ("q", vp), ("k_cache", vp), ("v_cache", vp), ("out", vp), ("lse", vp),
        ("block_table", vp), ("kv_start", vp), ("row_seq", vp), ("seq_lens", vp), ("key_lo", vp),
        ("workspace", vp), ("workspace_bytes", sz),
        ("num_rows", i64),
        ("num_q_heads", i32), ("num_kv_heads", i32), ("head_size", i32), ("block_size", i32),
        ("window_left", i32), ("max_seq_len", i32), ("n_split", i32), ("dtype", i32),
        ("phases", i32), ("flags", i32), ("scale", f32),
        ("q_stride_row", i64), ("q_stride_head", i64),
        ("out_stride_row", i64), ("out_stride_head", i64),
        ("kv_stride_block", i64), ("kv_stride_row", i64), ("kv_stride_head", i64),
        ("block_table_stride", i64),
        ("new_key", vp), ("new_value", vp), ("new_slot_mapping", vp),
        ("new_key_stride_row", i64), ("new_key_stride_head", i64),
        ("new_value_stride_row", i64), ("new_value_stride_head", i64),
        ("stream", vp), ("k_scale", vp), ("v_scale", vp), ("kv_quant", i32),
        ("k_scale_tensor", f32), ("v_scale_tensor", f32),
        ("meta_k", vp), ("meta_v", vp), ("meta_len", i32), ("meta_stride_row", i64), ("meta_stride_head", i64),
        ("profile_start_event", vp), ("profile_stop_event", vp),
        ("softcap", f32), ("alibi_slopes", vp), ("meta_bias_row0", i64), ("meta_bias_rows", i64),
    ]


class GlaRecurrentArgs(C.Structure):
    _fields_ = [
        ("q", vp), ("k", vp), ("v", vp), ("g", vp), ("state", vp), ("out", vp), ("slot_idx", vp),
        ("batch", i64), ("num_heads", i32), ("seq_len", i32), ("head_dim", i32),
        ("dtype", i32), ("g_dtype", i32), ("state_dtype", i32), ("scale", f32),
        ("q_stride_b", i64), ("q_stride_h", i64), ("q_stride_t", i64),
        ("k_stride_b", i64), ("k_stride_h", i64), ("k_stride_t", i64),
        ("v_stride_b", i64), ("v_stride_h", i64), ("v_stride_t", i64),
        ("g_stride_b", i64), ("g_stride_h", i64), ("g_stride_t", i64),
        ("out_stride_b", i64), ("out_stride_h", i64), ("out_stride_t", i64),
        ("state_stride_slot", i64), ("state_stride_head", i64),
        ("num_slots", i64), ("stream", vp), ("cu_seqlens", vp), ("flags", i32), ("q_heads_per_state", i32),
        ("profile_start_event", vp), ("profile_stop_event", vp),
    ]


class WindowShiftArgs(C.Structure):
    _fields_ = [
        ("src", vp), ("dst", vp), ("fresh", vp),
        ("planes", i64), ("keep_rows", i64), ("src_row0", i64), ("dst_row0", i64), ("n_new", i64),
        ("row_bytes", i64), ("src_stride_plane_bytes", i64), ("dst_stride_plane_bytes", i64),
        ("fresh_stride_plane_bytes", i64), ("fresh_stride_row_bytes", i64), ("stream", vp),
    ]


class SwaPrefillArgs(C.Structure):
    _fields_ = [
        ("q", vp), ("k", vp), ("v", vp), ("out", vp),
        ("block_table", vp), ("kv_start", vp), ("key_lo", vp), ("cu_seqlens_q", vp), ("seq_lens_k", vp),
        ("tile_seq", vp), ("tile_q0", vp),
        ("num_tiles", i64),
        ("num_q_heads", i32), ("num_kv_heads", i32), ("head_size", i32), ("block_size", i32),
        ("window_left", i32), ("dtype", i32), ("scale", f32),
        ("q_stride_row", i64), ("q_stride_head", i64),
        ("out_stride_row", i64), ("out_stride_head", i64),
        ("kv_stride_block", i64), ("kv_stride_row", i64), ("kv_stride_head", i64),
        ("block_table_stride", i64),
        ("stream", vp), ("lse", vp), ("k_scale", vp), ("v_scale", vp), ("kv_quant", i32),
        ("k_scale_tensor", f32), ("v_scale_tensor", f32),
        ("meta_k", vp), ("meta_v", vp), ("meta_len", i32), ("meta_stride_row", i64), ("meta_stride_head", i64),
        ("softcap", f32), ("alibi_slopes", vp), ("meta_bias_row0", i64), ("meta_bias_rows", i64),
    ]


class LseMergeArgs(C.Structure):
    _fields_ = [
        ("out", vp), ("lse", vp), ("block_out", vp), ("block_lse", vp),
        ("rows", i64), ("heads", i32), ("head_size", i32), ("dtype", i32),
        ("out_stride_row", i64), ("out_stride_head", i64),
        ("block_out_stride_row", i64), ("block_out_stride_head", i64),
        ("stream", vp),
    ]


class KvAppendInt8Args(C.Structure):
    _fields_ = [
        ("key", vp), ("value", vp), ("k_cache", vp), ("v_cache", vp), ("k_scale", vp), ("v_scale", vp),
        ("slot_mapping", vp), ("num_tokens", i64),
        ("num_kv_heads", i32), ("head_size", i32), ("block_size", i32), ("dtype", i32),
        ("key_stride_token", i64), ("key_stride_head", i64),
        ("value_stride_token", i64), ("value_stride_head", i64),
        ("cache_stride_block", i64), ("cache_stride_row", i64), ("cache_stride_head", i64),
        ("stream", vp),
    ]


class KvAppendFp8Args(C.Structure):
    _fields_ = [
        ("key", vp), ("value", vp), ("k_cache", vp), ("v_cache", vp), ("slot_mapping", vp), ("num_tokens", i64),
        ("num_kv_heads", i32), ("head_size", i32), ("block_size", i32), ("dtype", i32),
        ("key_stride_token", i64), ("key_stride_head", i64),
        ("value_stride_token", i64), ("value_stride_head", i64),
        ("cache_stride_block", i64), ("cache_stride_row", i64), ("cache_stride_head", i64),
        ("k_scale", f32), ("v_scale", f32),
        ("stream", vp),
    ]


class QuantizeSymArgs(C.Structure):
    _fields_ = [
        ("in_", vp), ("out", vp), ("rows", i64), ("heads", i32), ("head_size", i32), ("dtype", i32),
        ("in_stride_row", i64), ("in_stride_head", i64), ("out_stride_row", i64), ("out_stride_head", i64),
        ("stream", vp),
    ]


class WindowAdvanceArgs(C.Structure):
    _fields_ = [
        ("n_tokens", vp), ("lo", vp), ("hi", vp), ("ring", vp), ("free_stack", vp), ("free_top", vp),
        ("slot_mapping", vp), ("seq_lens", vp), ("block_tables", vp), ("status", vp),
        ("batch", i64),
        ("ring_blocks", i32), ("block_size", i32), ("window_left", i32), ("table_width", i32), ("num_blocks", i32),
        ("stream", vp),
    ]


# name -> (restype, argtypes); every symbol include/sbcache.h declares
EXPORTS = {
    "sb_abi_version": (C.c_int, []),
    "sb_last_error": (C.c_char_p, []),
    "sb_kv_append": (C.c_int, [C.POINTER(KvAppendArgs)]),
    "sb_swa_decode_auto_split": (i32, [i64, i32, i32, i32]),
    "sb_swa_decode_workspace_bytes": (sz, [i64, i32, i32, i32]),
    "sb_swa_decode_prefer_balanced": (i32, [C.POINTER(i32), i64, i32, i32]),
    "sb_swa_decode": (C.c_int, [C.POINTER(SwaDecodeArgs)]),
    "sb_swa_decode_static": (C.c_int, [C.POINTER(SwaDecodeArgs)]),
    "sb_gla_recurrent": (C.c_int, [C.POINTER(GlaRecurrentArgs)]),
    "sb_gla_gate_range_hits": (C.c_int, [C.POINTER(C.c_int64), C.c_int32]),
    "sb_copy_blocks": (C.c_int, [vp, vp, i64, i64, i64, vp]),
    "sb_window_shift": (C.c_int, [C.POINTER(WindowShiftArgs)]),
    "sb_swa_prefill": (C.c_int, [C.POINTER(SwaPrefillArgs)]),
    "sb_window_advance": (C.c_int, [C.POINTER(WindowAdvanceArgs)]),
    "sb_lse_merge": (C.c_int, [C.POINTER(LseMergeArgs)]),
    "sb_kv_append_int8": (C.c_int, [C.POINTER(KvAppendInt8Args)]),
    "sb_quantize_sym": (C.c_int, [C.POINTER(QuantizeSymArgs)]),
    "sb_kv_append_fp8": (C.c_int, [C.POINTER(KvAppendFp8Args)]),
    "sb_fp8_round": (C.c_int, [vp, vp, i64, i64, i64, i64, i32, f32, vp]),
    "sb_stream_copy": (C.c_int, [vp, vp, i64, vp]),
    "sb_stream_capture_id": (C.c_int, [vp, C.POINTER(C.c_uint64)]),
}

_lib: Optional[C.CDLL] = None


class NativeLibraryError(RuntimeError):
    pass


def lib() -> C.CDLL:
    """Load libsbcache.so once; raise NativeLibraryError if it is missing or stale."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or __graft_entry__.build()); there is no fallback path")
    try:
        handle = C.CDLL(LIB_PATH)
    except OSError as e:  # unresolved HIP runtime etc.
        raise NativeLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    for name, (res, args) in EXPORTS.items():
        try:
            fn = getattr(handle, name)
        except AttributeError as e:
            raise NativeLibraryError(f"{LIB_PATH} does not export {name}") from e
        fn.restype = res
        fn.argtypes = args
    got = handle.sb_abi_version()
    if got != ABI_VERSION:
        raise NativeLibraryError(f"{LIB_PATH} has ABI version {got}, this package needs {ABI_VERSION}")
    _lib = handle
    return handle


def last_error() -> str:
    return lib().sb_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    """Map a C-ABI return code onto the exception types the reference's callers see."""
    if rc == 0:
        return
    msg = f"{what}: {last_error()} (code {rc})"
    if rc == SB_ERR_INVALID:
        raise ValueError(msg)
    if rc == SB_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise NotImplementedError(f"dtype {dt} is not supported (bfloat16, float16, float32)") from None


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    """All tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("libsbcache kernels need tensors in GPU memory; got a "
                               f"{t.device} tensor (there is no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()
