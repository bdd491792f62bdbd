"""The CPU oracle under AddressSanitizer + UndefinedBehaviorSanitizer, and its threaded step under
ThreadSanitizer (host code only): the checker must not itself read out of bounds or race."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = [os.path.join(ROOT, "oracle", "selftest.c"), os.path.join(ROOT, "oracle", "adamw_oracle.c")]
BASE = ["gcc", "-O1", "-g", "-fno-math-errno", "-ffp-contract=off", "-fno-omit-frame-pointer"]


@pytest.mark.parametrize("name,flags", [
    ("asan_ubsan", ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan", "-static-libubsan"]),
    ("tsan", ["-fsanitize=thread", "-static-libtsan"])])
def test_oracle_under_sanitizers(tmp_path, name, flags):
    exe = str(tmp_path / name)
    build = subprocess.run(BASE + flags + ["-o", exe] + SRC + ["-lm", "-lpthread"], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="halt_on_error=1", TSAN_OPTIONS="halt_on_error=1")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    if name == "tsan" and run.returncode < 0 and not run.stdout and "ThreadSanitizer:" not in run.stderr:
        pytest.skip("the ThreadSanitizer runtime cannot start in this container (no report, signal %d)"
                    % -run.returncode)
    assert run.returncode == 0 and "selftest ok" in run.stdout, run.stdout + run.stderr
