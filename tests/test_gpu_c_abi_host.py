"""The C ABI called from a plain C++ host program: no Python, no torch in that process. The program
(tests/c_abi_host/host_check.cpp, built by __graft_entry__.build()) allocates with hipMalloc, calls
sb_kv_append, sb_swa_decode (two splits: workspace and merge included) and sb_gla_recurrent with the structs
of include/sbcache.h and checks the results against host loops in double precision: cache bytes exact,
attention within 2e-2, GLA state within 1e-4 relative."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_host_program_drives_the_library():
    exe = os.path.join(HERE, "c_abi_host", "host_check")
    assert os.path.exists(exe), "tests/c_abi_host/host_check is built by __graft_entry__.build()"
    run = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, run.stdout + run.stderr
    assert run.stdout.strip().endswith("ok"), run.stdout
    assert "attention (head size 128, 28 : 4 heads): max abs error" in run.stdout
    assert "attention (head size 64, 12 : 4 heads): max abs error" in run.stdout
    assert "gla: state max abs error" in run.stdout
