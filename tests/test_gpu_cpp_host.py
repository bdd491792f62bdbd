"""Runs the C++ host-side test (the reference-shaped AdamWOptimizer / clip_grad_norm_ / launch_adamw_*
mirror in rl.cu_amd/host) on the GPU.  The binaries are built beforehand by __graft_entry__.build(); make runs
again here every time, so that a binary older than the headers it was built from is never what gets tested (an
up-to-date one costs nothing)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "test_adamw_host.bin")


def test_cpp_host_mirror(torch_gpu):
    subprocess.run(["make", "-C", os.path.dirname(EXE), "-s"], check=True)
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    print(res.stdout)
    print(res.stderr)
    assert res.returncode == 0, res.stdout + res.stderr
    assert res.stdout.count("[PASS]") == 13 and "[FAIL]" not in res.stdout


def test_reference_call_sites_compile_unchanged_and_match_the_oracle(torch_gpu):
    """tests/cpp/test_reference_callsites.cpp: structs named Qwen3Model / Qwen3Gradients with only the fields the
    path reads, the lines of the reference's trainer.h:280-286 and GRPO_trainer.h:508-514 unchanged, every result
    bit-identical to the oracle replaying the reference's order of operations."""
    exe = os.path.join(ROOT, "tests", "cpp", "test_reference_callsites.bin")
    subprocess.run(["make", "-C", os.path.dirname(exe), "-s"], check=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=200)
    print(res.stdout)
    print(res.stderr)
    assert res.returncode == 0, res.stdout + res.stderr
    assert res.stdout.count("[PASS]") == 7 and "[FAIL]" not in res.stdout
    src = open(os.path.join(ROOT, "tests", "cpp", "test_reference_callsites.cpp")).read()
    for line in ("grad_norm = clip_grad_norm_(grads_, config_.max_grad_norm);", "optimizer_.step(grads_);",
                 "optimizer_(model, config.base_lr, config.beta1, config.beta2,"):
        assert line in src


def test_smoke_entry(torch_gpu):
    import __graft_entry__ as entry
    entry.smoke()
