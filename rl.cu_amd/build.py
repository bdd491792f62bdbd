"""Builds librlx_adamw.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
import hashlib
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "csrc", "rlx_adamw.hip")
OUT = os.path.join(HERE, "librlx_adamw.so")

# -ffp-contract=off: every FP32 operation of the update rounds once, as in the CPU restatement
# the results are checked against.  Packed FP32 instructions are switched off for device code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


HEADER = os.path.join(ROOT, "include", "rlx_adamw.h")
STAMP = OUT + ".srchash"


def source_hash():
    """Hash of everything the library is built from (kernel source, C header, compiler flags)."""
    h = hashlib.sha256()
    for path in (SRC, HEADER):
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def is_current():
    """True if the built library was made from the sources as they are now."""
    try:
        return os.path.exists(OUT) and open(STAMP).read().strip() == source_hash()
    except OSError:
        return False


def is_stale():
    """True if the library carries a source stamp and the stamp differs from the sources in the tree.  A library
    without a stamp was built by other means (the documented hipcc line, CMake) and is not judged here."""
    try:
        return os.path.exists(OUT) and os.path.exists(STAMP) and open(STAMP).read().strip() != source_hash()
    except OSError:
        return False


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def build_library(verbose=False):
    """Compiles the library every time it is called; returns the path of the .so."""
    cmd = [hipcc_path()] + HIPCC_FLAGS + ["-I", os.path.join(ROOT, "include"), "-o", OUT + ".tmp", SRC]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err)
    os.replace(OUT + ".tmp", OUT)
    with open(STAMP, "w") as f:
        f.write(source_hash() + "\n")
    return OUT


if __name__ == "__main__":
    print(build_library(verbose=True))
