"""Pins the oracle's AdamW update: against the CPU loops of the reference's own test
(tests/test_adamw.cu:194-206 and :276-293, restated with numpy FP32 scalars), against
torch.optim.AdamW (same mathematics, different rounding order), and against closed forms."""
import numpy as np
import pytest

B1, B2, EPS = 0.9, 0.999, 1e-8


def f32(x):
    return np.float32(x)


def _ref_test_loop_fp16(w0, g, lr, wd):
    """tests/test_adamw.cu:283-292: step 1, division by the bias corrections."""
    b1, b2, lr, wd, eps = f32(B1), f32(B2), f32(lr), f32(wd), f32(EPS)
    bc1, bc2 = f32(1) - b1, f32(1) - b2
    mi = (f32(1) - b1) * g
    vi = (f32(1) - b2) * g * g
    m_hat = mi / bc1
    v_hat = vi / bc2
    return w0 * (f32(1) - lr * wd) - lr * m_hat / (np.sqrt(v_hat) + eps)


def test_step1_fp16_against_reference_test_loop(O):
    """Case 2 of the reference's test: q_proj-sized tensor (2,097,152), lr=1e-3, wd=0.01.  Its
    pass criteria: master max abs err < 1e-6 and FP16 results identical; here the second is
    'at most 1 ulp, on a vanishing share', because the loop divides where the kernel
    multiplies by a host reciprocal."""
    n = 2048 * 1024
    p = O.fill_f16(n, 21, 0.0, 0.02)
    g = O.fill_f16(n, 22, 0.0, 1e-3)
    w0, gf = O.h2f(p), O.h2f(g)
    want = _ref_test_loop_fp16(w0, gf, 1e-3, 0.01).astype(np.float32)
    master = w0.copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    bc1, bc2 = O.bias_correction(B1, 1), O.bias_correction(B2, 1)
    O.adamw_fp16(master, p, g, m, v, 1e-3, B1, B2, EPS, 0.01, bc1, bc2)
    assert np.abs(master - want).max() < 1e-6
    assert np.array_equal(p, O.f2h(master))                      # model weight is f2h(master) exactly
    mism = p != O.f2h(want)
    assert mism.mean() < 1e-3
    a, b = O.h2f(p[mism]), O.h2f(O.f2h(want)[mism])
    assert (np.abs(a - b) <= np.spacing(np.abs(b).astype(np.float16)).astype(np.float32)).all()
    # moments as the loop computes them (exact: same two operations)
    assert np.array_equal(m, ((f32(1) - f32(B1)) * gf).astype(np.float32))
    assert np.array_equal(v, ((f32(1) - f32(B2)) * gf * gf).astype(np.float32))


def test_step1_fp32_against_reference_test_loop(O):
    """Case 1 of the reference's test: final_norm (1024 FP32 weights), lr=1e-3, no decay; max abs err < 1e-6."""
    n = 1024
    w0 = O.fill_f32(n, 31, 1.0, 0.05)
    g = O.fill_f32(n, 32, 0.0, 1e-2)
    want = _ref_test_loop_fp16(w0, g, 1e-3, 0.0)
    w = w0.copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    O.adamw_fp32(w, g, m, v, 1e-3, B1, B2, EPS, 0.0, O.bias_correction(B1, 1), O.bias_correction(B2, 1))
    assert np.abs(w - want).max() < 1e-6


def test_against_torch_adamw_ten_steps(O):
    """torch.optim.AdamW (decoupled decay, bias correction) on FP32 CPU tensors: the same
    mathematics rounded in another order, so agreement to a few FP32 ulps of the state.
    The betas are exactly representable in FP32: torch forms 1 - beta in double, the reference
    in FP32 (`1.0f - beta2`, adamw.cu:27), which for beta2 = 0.999 differ by 1.3e-5 relative."""
    import torch
    n = 100_000
    b1, b2 = 0.875, 1.0 - 2.0 ** -8
    w0 = O.fill_f32(n, 41, 0.0, 0.02)
    lr, wd = 1e-3, 0.01
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.AdamW([p], lr=lr, betas=(b1, b2), eps=EPS, weight_decay=wd, foreach=False, fused=False)
    w = w0.copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(1, 11):
        g = O.fill_f32(n, 100 + step, 0.0, 1e-3)
        p.grad = torch.from_numpy(g.copy())
        opt.step()
        O.adamw_fp32(w, g, m, v, lr, b1, b2, EPS, wd, O.bias_correction(b1, step), O.bias_correction(b2, step))
        st = opt.state[p]
        tm, tv = st["exp_avg"].numpy(), st["exp_avg_sq"].numpy()
        assert np.abs(m - tm).max() <= 4e-7 * np.abs(tm).max()
        assert (np.abs(v - tv) <= 1e-6 * np.abs(tv) + 1e-30).all()
        assert np.abs(w - p.detach().numpy()).max() <= 2e-6 * lr * step + 1e-8
    # a dropped bias correction, a wrong sign or coupled decay would be orders of magnitude outside
    assert np.abs(w - w0).max() > 5 * lr


def test_closed_forms(O):
    n = 4096
    w0 = O.fill_f32(n, 51, 0.5, 0.1)
    zeros = np.zeros(n, np.float32)
    # zero gradient, zero moments, no decay: nothing moves, bit for bit (frozen embedding)
    w, m, v = w0.copy(), zeros.copy(), zeros.copy()
    for t in range(1, 4):
        O.adamw_fp32(w, zeros, m, v, 1e-3, B1, B2, EPS, 0.0, O.bias_correction(B1, t), O.bias_correction(B2, t))
    assert np.array_equal(w, w0) and not m.any() and not v.any()
    # zero gradient with decay: w0 * (1 - lr*wd)^t, rounded once per step
    w = w0.copy()
    want = w0.copy()
    factor = f32(1) - f32(1e-2) * f32(0.1)
    for t in range(1, 6):
        O.adamw_fp32(w, zeros, m, v, 1e-2, B1, B2, EPS, 0.1, O.bias_correction(B1, t), O.bias_correction(B2, t))
        want = (want * factor).astype(np.float32)
    assert np.array_equal(w, want)
    assert np.allclose(w, w0 * (1 - 1e-2 * 0.1) ** 5, rtol=1e-6)
    # first step with |g| >> eps and no decay is a sign step of size lr
    g = O.fill_f32(n, 52, 0.0, 1.0)
    g[np.abs(g) < 1e-3] = 1e-3
    w, m, v = w0.copy(), zeros.copy(), zeros.copy()
    O.adamw_fp32(w, g, m, v, 1e-3, B1, B2, EPS, 0.0, O.bias_correction(B1, 1), O.bias_correction(B2, 1))
    assert np.abs((w - w0) + 1e-3 * np.sign(g)).max() < 1e-3 * 1e-4 + 1e-7


def test_moments_do_not_depend_on_lr_wd_eps(O):
    n = 10_000
    g = O.fill_f16(n, 61, 0.0, 1e-3)
    outs = []
    for lr, wd, eps in ((1e-5, 0.01, 1e-8), (3e-2, 0.3, 1e-3)):
        p = O.fill_f16(n, 62, 0.0, 0.02)
        m, v = O.fill_f32(n, 63, 0.0, 1e-4), O.fill_f32(n, 64, 1e-8, 1e-8, flags=O.FILL_ABS)
        O.adamw_fp16(None, p, g, m, v, lr, B1, B2, eps, wd, 0.5, 0.25)
        outs.append((m, v))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])


def test_elementwise_independence(O):
    """Any slicing or permutation of the tensor gives the same value per element."""
    n = 50_000
    rng = np.random.default_rng(3)
    perm = rng.permutation(n)
    p, g = O.fill_f16(n, 71, 0.0, 0.02), O.fill_f16(n, 72, 0.0, 1e-3)
    m, v = O.fill_f32(n, 73, 0.0, 1e-4), O.fill_f32(n, 74, 1e-8, 1e-8, flags=O.FILL_ABS)
    args = (1e-4, B1, B2, EPS, 0.01, O.bias_correction(B1, 7), O.bias_correction(B2, 7))
    a = [x.copy() for x in (p, g, m, v)]
    O.adamw_fp16(None, a[0], a[1], a[2], a[3], *args)
    b = [np.ascontiguousarray(x[perm]) for x in (p, g, m, v)]
    O.adamw_fp16(None, b[0], b[1], b[2], b[3], *args)
    for x, y in zip(a, b):
        assert np.array_equal(x[perm], y)
    c = [x.copy() for x in (p, g, m, v)]
    for lo, hi in ((0, 1), (1, 4097), (4097, n)):
        O.adamw_fp16(None, c[0][lo:hi], c[1][lo:hi], c[2][lo:hi], c[3][lo:hi], *args)
    for x, y in zip(a, c):
        assert np.array_equal(x, y)


def test_master_mode_and_masterless_mode(O):
    """With a master copy the FP16 weight is never read (Q: adamw.cu:35-39); without one the FP16
    weight is the source of truth.  The two agree for one step when master == h2f(weight)."""
    n = 8192
    p0, g = O.fill_f16(n, 81, 0.0, 0.02), O.fill_f16(n, 82, 0.0, 1e-3)
    args = (1e-3, B1, B2, EPS, 0.01, O.bias_correction(B1, 1), O.bias_correction(B2, 1))
    pa, ma, va = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    O.adamw_fp16(None, pa, g, ma, va, *args)
    garbage = np.full(n, 0x3C00, np.uint16)
    master, mb, vb = O.h2f(p0), np.zeros(n, np.float32), np.zeros(n, np.float32)
    O.adamw_fp16(master, garbage, g, mb, vb, *args)
    assert np.array_equal(garbage, pa) and np.array_equal(ma, mb) and np.array_equal(va, vb)
    assert np.array_equal(O.f2h(master), garbage)


def test_bias_correction(O):
    # step 1 gives 1 - beta exactly, as the reference's test assumes (tests/test_adamw.cu:196-197)
    assert O.bias_correction(B1, 1) == float(f32(1) - f32(B1))
    assert O.bias_correction(B2, 1) == float(f32(1) - f32(B2))
    for t in (2, 10, 100, 1000, 100000):
        for b in (B1, B2):
            want = 1.0 - float(f32(b)) ** t        # beta is an FP32 value on the reference's host
            assert abs(O.bias_correction(b, t) - want) <= 2e-7 * max(want, 1e-3) + 1e-7
    assert O.bias_correction(B1, 100000) == 1.0


def test_optimizer_step_groups(O):
    """optimizer.h:119-147: step counter first; decay on projections only; embedding and FP32 norm
    pools get weight_decay 0 whatever the configured value."""
    n16, proj_n, n32 = 3000, 2000, 300
    pool16 = O.fill_f16(n16, 91, 0.0, 0.5)
    master = O.h2f(pool16)
    g16 = np.zeros(n16, np.uint16)
    pool32, g32 = O.fill_f32(n32, 92, 1.0, 0.1), np.zeros(n32, np.float32)
    m16, v16 = np.zeros(n16, np.float32), np.zeros(n16, np.float32)
    m32, v32 = np.zeros(n32, np.float32), np.zeros(n32, np.float32)
    before16, before32 = master.copy(), pool32.copy()
    step = O.optimizer_step(master, pool16, g16, m16, v16, proj_n, pool32, g32, m32, v32,
                            1e-2, B1, B2, EPS, 0.1, 0)
    assert step == 1
    factor = f32(1) - f32(1e-2) * f32(0.1)
    assert np.array_equal(master[:proj_n], (before16[:proj_n] * factor).astype(np.float32))
    assert np.array_equal(master[proj_n:], before16[proj_n:])
    assert np.array_equal(pool32, before32)
    assert O.optimizer_step(master, pool16, g16, m16, v16, proj_n, pool32, g32, m32, v32,
                            1e-2, B1, B2, EPS, 0.1, step) == 2


@pytest.mark.parametrize("n", [0, -3])
def test_non_positive_n_is_a_no_op(O, n):
    # adamw.cu:49,99: returns before touching anything, even null pointers
    O.lib.orc_adamw_fp16(None, None, None, None, None, n, 1e-3, B1, B2, EPS, 0.0, 0.1, 0.001)
    O.lib.orc_adamw_fp32(None, None, None, None, n, 1e-3, B1, B2, EPS, 0.0, 0.1, 0.001)


def test_threaded_step_matches_single_thread(O):
    n = 100_003
    p, g = O.fill_f16(n, 95, 0.0, 0.02), O.fill_f16(n, 96, 0.0, 5e-3)
    args = (1e-3, B1, B2, EPS, 0.01, O.bias_correction(B1, 3), O.bias_correction(B2, 3))
    pa, ma, va = p.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    ga = g.copy()
    norm, scale = O.clip_grad_norm(ga, None, 1.0)
    O.adamw_fp16(None, pa, ga, ma, va, *args)
    pb, mb, vb = p.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    norm_b = O.step_fp16_threaded(None, pb, g, mb, vb, *args, 1.0, 5)
    assert abs(norm_b - norm) <= 1e-6 * norm and norm > 1.0
    assert np.array_equal(pa, pb) and np.array_equal(ma, mb) and np.array_equal(va, vb)


def _fma(a, b, c):
    """float32 fused multiply-add: the product of two float32 values is exact in float64; the sum is rounded to
    float64 and then to float32 (a double rounding that can differ from a true FMA in rare ties, which is far
    below what this test measures)."""
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)


def test_tolerances_cover_a_reference_binary_built_with_fma_contraction(O):
    """The reference's CUDA kernel is compiled with nvcc's default -fmad=true, so its binary most likely contracts
    the multiply-adds of src/kernels/adamw.cu:25-36 into FMAs; this path (kernel and oracle) rounds every operation
    once.  Which of the two the reference's binary does cannot be observed without its hardware; what can be shown
    is that the stated tolerances (FP32 moments 1e-6 relative, FP16 weights 1 ulp) cover the difference (for the
    first moment relative to the largest terms it has added up, since the sum itself can cancel): the
    configuration of config 0 (1,048,576 params, 10 steps, fresh gradients) replayed with every contractible
    multiply-add fused, against the oracle."""
    n = 1 << 20
    lr, wd = f32(1e-5), f32(0.01)
    b1, b2, eps, one = f32(B1), f32(B2), f32(EPS), f32(1)
    p = O.fill_f16(n, 41, 0.0, 0.02)
    p_fma = p.copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    m_f, v_f = m.copy(), v.copy()
    worst_m = worst_v = 0.0
    m_scale = np.zeros(n, np.float32)
    for step in range(1, 11):
        gbits = O.fill_f16(n, 50 + step, 0.0, 1e-3)
        g = O.h2f(gbits)
        bc1, bc2 = O.bias_correction(B1, step), O.bias_correction(B2, step)
        m_prev = m.copy()
        O.adamw_fp16(None, p, gbits, m, v, lr, B1, B2, EPS, wd, bc1, bc2)
        # the same step with a*b + c*d -> fma(a, b, c*d), 1 - lr*wd -> fma(-lr, wd, 1), w*x - y -> fma(w, x, -y)
        bc1_inv, bc2_inv = one / f32(bc1), one / f32(bc2)
        w = O.h2f(p_fma)
        m_f = _fma(np.full(n, b1), m_f, (one - b1) * g)
        v_f = _fma((one - b2) * g, g, b2 * v_f)
        m_hat, v_hat = m_f * bc1_inv, v_f * bc2_inv
        decay = _fma(np.full(n, -lr), np.full(n, wd), np.full(n, one))
        upd = lr * m_hat / (np.sqrt(v_hat) + eps)
        p_fma = O.f2h(_fma(w, decay, -upd))
        # v is a sum of non-negative terms: plain relative error.  m is a sum of terms of either sign that can cancel
        # to nearly nothing, and a rounding difference made while the terms were large stays in the element when
        # they have become small: its error is measured against the largest terms the element has added so far
        nz = v != 0
        worst_v = max(worst_v, float((np.abs(v_f - v)[nz] / v[nz]).max()))
        m_scale = np.maximum(m_scale, np.abs(b1 * m_prev) + np.abs((one - b1) * g))
        nzt = m_scale != 0
        worst_m = max(worst_m, float((np.abs(m_f - m)[nzt] / m_scale[nzt]).max()))
        ulp = np.abs(p.astype(np.int32) - p_fma.astype(np.int32))
        same_sign = (p & 0x8000) == (p_fma & 0x8000)
        assert ulp[same_sign].max() <= 1 and (ulp[~same_sign] <= 1).all(), step      # +-0 against each other at most
    assert worst_m <= 1e-6 and worst_v <= 1e-6, (worst_m, worst_v)


def test_threaded_list_step_equals_per_tensor_steps(O):
    """The CPU baseline's step over a tensor list (one split of the concatenated index space over the threads)
    gives, for any thread count, the bits of the plain per-tensor update; with clipping, the norm is within the
    path's 1e-5 of the FP64 sum and the scaled, re-rounded gradients are the ones the update sees."""
    sizes = [128, 1024, 5000, 7, 65536, 300]
    off, total = [], 0
    for n in sizes:
        off.append(total)
        total += (n + 127) // 128 * 128
    p, g = O.fill_f16(total, 1, 0.0, 0.02), O.fill_f16(total, 2, 0.0, 5e-3)
    m, v = O.fill_f32(total, 3, 0.0, 1e-4), O.fill_f32(total, 4, 1e-8, 1e-8, flags=O.FILL_ABS)
    args = (1e-3, 0.9, 0.999, 1e-8, 0.01, 0.1, 0.001)
    for max_norm in (0.0, 0.01):
        ref = [x.copy() for x in (p, m, v)]
        ssq = sum(O.sum_sq_half(np.ascontiguousarray(g[o: o + n])) for o, n in zip(off, sizes))
        scale, norm = O.clip_scale(np.float32(ssq), max_norm) if max_norm > 0 else (None, 0.0)
        for o, n in zip(off, sizes):
            parts = [np.ascontiguousarray(x[o: o + n]) for x in ref]
            O.adamw_fp16(None, parts[0], np.ascontiguousarray(g[o: o + n]), parts[1], parts[2], *args,
                         clip_scale=scale if max_norm > 0 and norm > max_norm else None)
            for x, part in zip(ref, parts):
                x[o: o + n] = part
        for threads in (1, 3, 16):
            q = [x.copy() for x in (p, g, m, v)]
            got = O.step_list_fp16_threaded(q[0], q[1], q[2], q[3], off, off, sizes, *args, max_norm, threads)
            assert np.array_equal(q[0], ref[0]) and np.array_equal(q[1], g), threads
            assert np.array_equal(q[2].view(np.uint32), ref[1].view(np.uint32)), threads
            assert np.array_equal(q[3].view(np.uint32), ref[2].view(np.uint32)), threads
            assert abs(got - norm) <= 1e-5 * max(norm, 1e-30), threads
