"""The learning-rate scheduler that feeds set_lr (include/training/lr_scheduler.h:10-57): golden
vectors written by the reference's own class, the reference's own test compiled against this
repository's header, and the Python mirror."""
import json
import os
import struct
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = json.load(open(os.path.join(ROOT, "tests", "golden", "lr_schedule.json")))
CASES = {
    "constant_1e-4": ("constant", 1e-4, 0),
    "constant_1e-3_warmup10": ("constant", 1e-3, 10),
    "constant_1e-5_warmup1": ("constant", 1e-5, 1),
    "cosine_1e-3_1e-5_w0_t100": ("cosine", 1e-3, 1e-5, 0, 100),
    "cosine_1e-3_1e-4_w10_t110": ("cosine", 1e-3, 1e-4, 10, 110),
    "cosine_1e-5_0_w50_t2000": ("cosine", 1e-5, 0.0, 50, 2000),
    "cosine_total_equals_warmup": ("cosine", 3e-4, 3e-5, 10, 10),
    "cosine_total_below_warmup": ("cosine", 3e-4, 3e-5, 10, 5),
    "default_constructed": ("default",),
}


def f32bits(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def test_golden_is_complete():
    assert set(GOLDEN) == set(CASES) and sum(len(v) for v in GOLDEN.values()) == 2450


@pytest.mark.parametrize("name", sorted(CASES))
def test_python_mirror_matches_reference_vectors(host, name):
    s = host.LRScheduler()
    c = CASES[name]
    if c[0] == "constant":
        s.init_constant(c[1], c[2])
    elif c[0] == "cosine":
        s.init_cosine(*c[1:])
    got = [f32bits(s.get_lr(i)) for i in range(len(GOLDEN[name]))]
    assert got == GOLDEN[name]


def test_cpp_mirror_matches_reference_vectors():
    """oracle/lr_dump.cpp compiled against rl.cu_amd/host/training/lr_scheduler.h."""
    exe = os.path.join(ROOT, "oracle", "lr_dump_mirror")
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-s", "lr_dump_mirror"], check=True)
    out = json.loads(subprocess.run([exe], check=True, capture_output=True, text=True).stdout)
    assert out == GOLDEN


def test_known_values(host):
    """The values the reference's test spells out (tests/test_lr_scheduler.cpp: warm-up of 10 steps to 1e-3
    starts at 1e-4 and reaches 5e-4 at step 4; cosine starts at base and ends at min)."""
    s = host.LRScheduler()
    s.init_constant(1e-3, 10)
    assert abs(s.get_lr(0) - 1e-4) < 1e-9 and abs(s.get_lr(4) - 5e-4) < 1e-9 and abs(s.get_lr(10) - 1e-3) < 1e-9
    s.init_cosine(1e-3, 1e-5, 0, 100)
    assert abs(s.get_lr(0) - 1e-3) < 1e-9 and abs(s.get_lr(50) - 5.05e-4) < 1e-7 and s.get_lr(100) == s.get_lr(500)
    assert f32bits(s.get_lr(100)) == f32bits(1e-5)


def test_reference_test_against_this_header():
    """tests/test_lr_scheduler.cpp of the reference, compiled with this repository's header in place of
    the reference's (built by `make -C oracle ref` where the reference tree is present)."""
    exe = os.path.join(ROOT, "oracle", "_ref", "test_lr_scheduler_mirror")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref is built only where the reference tree is present")
    res = subprocess.run([exe], capture_output=True, text=True)
    assert res.returncode == 0 and "[FAIL]" not in res.stdout and res.stdout.count("[PASS]") >= 5, res.stdout
    ref = subprocess.run([os.path.join(ROOT, "oracle", "_ref", "test_lr_scheduler_ref")], capture_output=True, text=True)
    assert ref.stdout == res.stdout
