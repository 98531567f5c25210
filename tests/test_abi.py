"""The C-ABI library loads and exports every symbol include/sbcache.h declares; argument
rejection that happens before any HIP call works without a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sbcache.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sb_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_all_exported(sb):
    names = declared_symbols()
    assert "sb_kv_append" in names and "sb_swa_decode" in names and "sb_gla_recurrent" in names
    lib = C.CDLL(sb._native.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/sbcache.h but not exported"
    assert set(names) == set(sb._native.EXPORTS), "ctypes table and header disagree"


def test_abi_version(sb):
    assert sb._native.lib().sb_abi_version() == sb._native.ABI_VERSION


def test_null_args_rejected(sb):
    L = sb._native.lib()
    assert L.sb_kv_append(None) == sb._native.SB_ERR_INVALID
    assert b"null" in L.sb_last_error()
    assert L.sb_swa_decode(None) == sb._native.SB_ERR_INVALID
    assert L.sb_gla_recurrent(None) == sb._native.SB_ERR_INVALID
    assert L.sb_window_shift(None) == sb._native.SB_ERR_INVALID


def test_bad_shapes_rejected_before_launch(sb):
    N = sb._native
    L = N.lib()
    a = N.SwaDecodeArgs(q=16, k_cache=16, v_cache=16, out=16, seq_lens=16, num_rows=1, num_q_heads=28,
                        num_kv_heads=4, head_size=48, block_size=16, scale=1.0, dtype=0)
    assert L.sb_swa_decode(C.byref(a)) == N.SB_ERR_UNSUPPORTED  # head sizes go from 32 to 256 in steps of 32
    a.head_size = 64
    a.kv_quant = N.SB_KV_INT8
    assert L.sb_swa_decode(C.byref(a)) == N.SB_ERR_UNSUPPORTED  # byte-code caches: 128 only
    a.kv_quant = N.SB_KV_NONE
    a.head_size = 128
    a.num_q_heads = 27
    assert L.sb_swa_decode(C.byref(a)) == N.SB_ERR_INVALID
    a.num_q_heads = 28
    a.scale = 0.0
    assert L.sb_swa_decode(C.byref(a)) == N.SB_ERR_INVALID
    a.scale = 1.0
    a.block_table = 16
    a.block_size = 24
    assert L.sb_swa_decode(C.byref(a)) == N.SB_ERR_INVALID
    a.block_size = 16
    a.n_split = 4  # needs a workspace
    assert L.sb_swa_decode(C.byref(a)) == N.SB_ERR_WORKSPACE
    g = N.GlaRecurrentArgs(q=16, k=16, v=16, g=16, state=16, out=16, batch=1, num_heads=1, seq_len=1, head_dim=64)
    assert L.sb_gla_recurrent(C.byref(g)) == N.SB_ERR_UNSUPPORTED
    # shared states: the group size must divide the query heads and stay within 8
    g = N.GlaRecurrentArgs(q=16, k=16, v=16, g=16, state=16, out=16, batch=1, num_heads=28, seq_len=1, head_dim=128,
                           state_dtype=N.SB_F32, state_stride_slot=4 * 16384, state_stride_head=16384)
    for bad in (3, 14, -1):
        g.q_heads_per_state = bad
        assert L.sb_gla_recurrent(C.byref(g)) == N.SB_ERR_INVALID


def test_auto_split_and_workspace(sb):
    L = sb._native.lib()
    n = L.sb_swa_decode_auto_split(64, 4, 32768, 4096)
    assert n == 4                                                   # 64 workgroups per split -> 256 = one per CU
    assert L.sb_swa_decode_auto_split(4096, 4, 32768, 4096) == 1
    assert L.sb_swa_decode_auto_split(1, 4, 300, 4096) == 1         # short windows are never split below 8 chunks
    assert L.sb_swa_decode_auto_split(1, 4, 1 << 20, -1) == 64      # capped
    assert L.sb_swa_decode_workspace_bytes(64, 28, 128, 1) == 0
    need = L.sb_swa_decode_workspace_bytes(64, 28, 128, 8)
    assert need >= 64 * 28 * 8 * 130 * 4


def test_balanced_split_policy_and_workspace(sb):
    """Host-side rule for the balanced split: even, window-saturated batches keep the fixed split,
    ragged ones take the balanced one; the workspace covers the partial numbering of both."""
    L = sb._native.lib()

    def prefer(lens, wl, n):
        return L.sb_swa_decode_prefer_balanced((C.c_int32 * len(lens))(*lens), len(lens), wl, n)

    assert prefer([4097 + 16 * i for i in range(64)], 4096, 4) == 0          # all rows fill the window
    assert prefer([32768] + [256] * 31, -1, 8) == 1                          # one long row among short ones
    assert prefer([100 + 120 * i for i in range(64)], -1, 4) == 1            # lengths spread over 100..7660
    assert prefer([5000] * 8, 4096, 1) == 1                                  # 8 unsplit rows leave 248 CUs idle
    assert prefer([], 4096, 4) == 0
    # even batches: the fixed split where rows x splits fills whole rounds of the 256 CUs, the balanced one
    # where the last round would be mostly empty or there would be several rounds
    auto = lambda rows: L.sb_swa_decode_auto_split(rows, 4, 8000, 4096)
    for rows, want in ((16, 0), (64, 0), (128, 0), (256, 0), (512, 0), (96, 1), (192, 1), (200, 1), (300, 1)):
        assert prefer([8000] * rows, 4096, auto(rows)) == want, rows
    assert prefer([8000] * 2048, 4096, 1) == 0                               # beyond the balanced kernel's row limit
    # the split count avoids a nearly empty extra round: 96 rows x 3 = 288 workgroups would run 256 + 32
    assert auto(96) == 5 and auto(80) == 3 and auto(48) == 5 and auto(32) == 8 and auto(128) == 2
    # balanced numbering: (workgroups, here one per CU = 256) + rows partial slots per head
    assert L.sb_swa_decode_workspace_bytes(48, 28, 128, 5) >= (256 + 48) * 28 * 130 * 4
    assert L.sb_swa_decode_workspace_bytes(64, 28, 128, 8) >= 64 * 8 * 28 * 130 * 4


def test_wrappers_refuse_cpu_tensors(sb):
    import torch
    k = torch.zeros(2, 4, 128, dtype=torch.bfloat16)
    cache = torch.zeros(4, 16, 4, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        sb.ops.kv_append(k, k, cache, cache, torch.zeros(2, dtype=torch.int64))
