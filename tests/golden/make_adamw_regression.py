"""Writes tests/golden/adamw_regression.json: a few hundred seeded elements pushed through the CPU
oracle (three FP16 steps with and without master copy and clip, two FP32 steps, norm and clip scale),
stored as bit patterns.  These are NOT reference outputs (the reference's AdamW is CUDA and cannot run
here): they freeze what the oracle computed once it had been pinned by tests/test_oracle_*.py, so that a
later change to the oracle, to the compiler flags or to the host CPU that moves a single bit is noticed."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import oracle as O  # noqa: E402


def run():
    n = 257
    out = {"n": n, "hyper": dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)}
    p = O.fill_f16(n, 1, 0.0, 0.02)
    p[:8] = [0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF]      # zeros, subnormals, extremes
    master = O.h2f(p)
    pm = p.copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    mm, vm = np.zeros(n, np.float32), np.zeros(n, np.float32)
    steps = []
    for step in (1, 2, 3):
        g = O.fill_f16(n, 10 + step, 0.0, 5e-3)
        g[:6] = [0x0000, 0x0001, 0x8001, 0x03FF, 0x7BFF, 0xFBFF]
        bc1, bc2 = O.bias_correction(0.9, step), O.bias_correction(0.999, step)
        norm, scale = O.clip_grad_norm(g.copy(), None, 0.05)
        O.adamw_fp16(None, p, g, m, v, 1e-3, 0.9, 0.999, 1e-8, 0.01, bc1, bc2, clip_scale=scale if step == 2 else None)
        O.adamw_fp16(master, pm, g, mm, vm, 1e-3, 0.9, 0.999, 1e-8, 0.01, bc1, bc2)
        steps.append(dict(step=step, g=g.tolist(), norm_bits=int(np.float32(norm).view(np.uint32)),
                          scale_bits=int(np.float32(scale).view(np.uint32)),
                          bc1_bits=int(np.float32(bc1).view(np.uint32)), bc2_bits=int(np.float32(bc2).view(np.uint32)),
                          p=p.tolist(), m=m.view(np.uint32).tolist(), v=v.view(np.uint32).tolist(),
                          p_master=pm.tolist(), master=master.view(np.uint32).tolist()))
    out["fp16"] = steps
    w = O.fill_f32(n, 21, 1.0, 0.05)
    m32, v32 = np.zeros(n, np.float32), np.zeros(n, np.float32)
    f32 = []
    for step in (1, 2):
        g = O.fill_f32(n, 30 + step, 0.0, 1e-2)
        O.adamw_fp32(w, g, m32, v32, 1e-3, 0.9, 0.999, 1e-8, 0.0, O.bias_correction(0.9, step),
                     O.bias_correction(0.999, step))
        f32.append(dict(step=step, w=w.view(np.uint32).tolist(), m=m32.view(np.uint32).tolist(),
                        v=v32.view(np.uint32).tolist()))
    out["fp32"] = f32
    out["p0"] = O.fill_f16(n, 1, 0.0, 0.02).tolist()
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "adamw_regression.json"), "w") as f:
        json.dump(run(), f, separators=(",", ":"))
        f.write("\n")
    print("written")
