"""Runs the C++ host-side test (the reference-shaped AdamWOptimizer / clip_grad_norm_ / launch_adamw_*
mirror in rl.cu_amd/host) on the GPU.  The binary is built beforehand by __graft_entry__.build()."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "test_adamw_host.bin")


def test_cpp_host_mirror(torch_gpu):
    if not os.path.exists(EXE):
        subprocess.run(["make", "-C", os.path.dirname(EXE), "-s"], check=True)
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    print(res.stdout)
    print(res.stderr)
    assert res.returncode == 0, res.stdout + res.stderr
    assert res.stdout.count("[PASS]") == 11 and "[FAIL]" not in res.stdout


def test_smoke_entry(torch_gpu):
    import __graft_entry__ as entry
    entry.smoke()
