"""GPU parity of the operator API (rlx_adamw_fp16 / rlx_adamw_fp32) against the CPU oracle."""
import numpy as np
import pytest

from util import HYPER, bits, check_state

pytestmark = pytest.mark.gpu


def _gen(O, B, torch, n, seed, std, mean=0.0):
    """The same seeded FP16 values on the device and on the host."""
    t = torch.empty(n, dtype=torch.float16, device="cuda:0")
    B.fill_f16(t.data_ptr(), n, seed, mean, std)
    return t, O.fill_f16(n, seed, mean, std)


@pytest.mark.parametrize("with_master", [False, True])
def test_config0_ten_steps(O, B, host, torch_gpu, with_master):
    """One flat tensor of 1,048,576 parameters, ten steps with fresh seeded gradients,
    p/m/v compared after every step (the reference's test_adamw layout with a CPU loop)."""
    torch = torch_gpu
    n = 1 << 20
    p_d, p_h = _gen(O, B, torch, n, 0x5EED0000, 0.02)
    torch.cuda.synchronize()
    assert np.array_equal(bits(p_d), p_h), "device and host generators disagree"
    m_d = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    v_d = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    m_h, v_h = np.zeros(n, np.float32), np.zeros(n, np.float32)
    w_d = w_h = None
    if with_master:
        w_d = torch.empty(n, dtype=torch.float32, device="cuda:0")
        B.check(B.fp16_to_fp32(w_d.data_ptr(), p_d.data_ptr(), n), "fp16_to_fp32")
        w_h = O.h2f(p_h)
    h = HYPER
    not_identical = 0
    for step in range(1, 11):
        g_d, g_h = _gen(O, B, torch, n, 0x6EAD0000 + step, 1e-3)
        bc1, bc2 = host.bias_correction(h["beta1"], step), host.bias_correction(h["beta2"], step)
        st = B.adamw_fp16(w_d.data_ptr() if with_master else None, p_d.data_ptr(), g_d.data_ptr(),
                          m_d.data_ptr(), v_d.data_ptr(), n, h["lr"], h["beta1"], h["beta2"], h["eps"],
                          h["wd"], bc1, bc2)
        assert st == B.OK
        O.adamw_fp16(w_h, p_h, g_h, m_h, v_h, h["lr"], h["beta1"], h["beta2"], h["eps"], h["wd"], bc1, bc2)
        torch.cuda.synchronize()
        not_identical += check_state(bits(p_d), bits(m_d), bits(v_d), p_h, m_h, v_h, "step %d" % step)
        if with_master:
            assert np.array_equal(bits(w_d), w_h)
    assert not_identical == 0, "within tolerance but not bit-identical: %d values" % not_identical


def test_fp32_variant(O, B, host, torch_gpu):
    torch = torch_gpu
    n = 65536 + 77
    w_d = torch.empty(n, dtype=torch.float32, device="cuda:0")
    g_d = torch.empty(n, dtype=torch.float32, device="cuda:0")
    B.fill_f32(w_d.data_ptr(), n, 1, 1.0, 0.01)
    B.fill_f32(g_d.data_ptr(), n, 2, 0.0, 1e-3)
    w_h, g_h = O.fill_f32(n, 1, 1.0, 0.01), O.fill_f32(n, 2, 0.0, 1e-3)
    m_d = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    v_d = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    m_h, v_h = np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(1, 4):
        bc1, bc2 = host.bias_correction(0.9, step), host.bias_correction(0.999, step)
        assert B.adamw_fp32(w_d.data_ptr(), g_d.data_ptr(), m_d.data_ptr(), v_d.data_ptr(), n,
                            1e-3, 0.9, 0.999, 1e-8, 0.0, bc1, bc2) == B.OK
        O.adamw_fp32(w_h, g_h, m_h, v_h, 1e-3, 0.9, 0.999, 1e-8, 0.0, bc1, bc2)
        torch.cuda.synchronize()
        assert check_state(bits(w_d), bits(m_d), bits(v_d), w_h, m_h, v_h) == 0


@pytest.mark.parametrize("n", [1, 7, 8, 9, 2047, 2048, 2049, 8191, 8192, 8193, 100003])
@pytest.mark.parametrize("offset", [0, 1, 3])
def test_ragged_sizes_and_misaligned_starts(O, B, host, torch_gpu, n, offset):
    """Tails shorter than one 128-bit access and tensors that do not start on a 16-byte boundary."""
    torch = torch_gpu
    pad = 64
    tot = n + offset + pad
    p_d, p_h = _gen(O, B, torch, tot, 5, 0.02)
    g_d, g_h = _gen(O, B, torch, tot, 6, 1e-3)
    m_d = torch.zeros(tot + 4, dtype=torch.float32, device="cuda:0")
    v_d = torch.zeros(tot + 4, dtype=torch.float32, device="cuda:0")
    m_h, v_h = np.zeros(tot, np.float32), np.zeros(tot, np.float32)
    bc1, bc2 = host.bias_correction(0.9, 1), host.bias_correction(0.999, 1)
    sl = slice(offset, offset + n)
    assert B.adamw_fp16(None, p_d.data_ptr() + 2 * offset, g_d.data_ptr() + 2 * offset,
                        m_d.data_ptr() + 4 * offset, v_d.data_ptr() + 4 * offset, n,
                        1e-3, 0.9, 0.999, 1e-8, 0.01, bc1, bc2) == B.OK
    O.adamw_fp16(None, p_h[sl], g_h[sl], m_h[sl], v_h[sl], 1e-3, 0.9, 0.999, 1e-8, 0.01, bc1, bc2)
    torch.cuda.synchronize()
    # everything outside [offset, offset+n) must be untouched, everything inside must match
    assert np.array_equal(bits(p_d), p_h)
    assert np.array_equal(bits(m_d)[:tot], m_h) and np.array_equal(bits(v_d)[:tot], v_h)
    assert not bits(m_d)[tot:].any()


def test_noop_and_errors(B, torch_gpu):
    torch = torch_gpu
    t = torch.zeros(64, dtype=torch.float32, device="cuda:0")
    h = torch.zeros(64, dtype=torch.float16, device="cuda:0")
    args = (1e-3, 0.9, 0.999, 1e-8, 0.01, 0.1, 0.001)
    # n <= 0 is a silent no-op (adamw.cu:49,99), even with null pointers
    assert B.adamw_fp16(None, None, None, None, None, 0, *args) == B.OK
    assert B.adamw_fp32(None, None, None, None, -5, *args) == B.OK
    assert B.adamw_fp16(None, None, h.data_ptr(), t.data_ptr(), t.data_ptr(), 8, *args) == B.ERR_INVALID_ARG
    assert B.adamw_fp16(None, h.data_ptr() + 1, h.data_ptr(), t.data_ptr(), t.data_ptr(), 8, *args) == B.ERR_MISALIGNED
    bad = (1e-3, 0.9, 0.999, 1e-8, 0.01, 0.0, 0.001)
    assert B.adamw_fp16(None, h.data_ptr(), h.data_ptr(), t.data_ptr(), t.data_ptr(), 8, *bad) == B.ERR_BAD_HYPER
    nan = (float("nan"), 0.9, 0.999, 1e-8, 0.01, 0.1, 0.001)
    assert B.adamw_fp32(t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 8, *nan) == B.ERR_BAD_HYPER
    torch.cuda.synchronize()
    assert not t.any().item() and not h.any().item()


def test_against_frozen_vectors(B, host, torch_gpu):
    """The operator API on the inputs of tests/golden/adamw_regression.json (zeros, FP16 subnormals and
    extremes among them) against the outputs stored there: three FP16 steps without and with master copy,
    two FP32 steps."""
    import json
    import os
    torch = torch_gpu
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    fx = json.load(open(os.path.join(root, "tests", "golden", "adamw_regression.json")))
    n, hy = fx["n"], fx["hyper"]

    def dev16(vals):
        return torch.from_numpy(np.array(vals, np.uint16).view(np.int16)).view(torch.float16).cuda()

    p0 = np.array(fx["p0"], np.uint16)
    p0[:8] = [0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF]
    pm = dev16(p0)
    master = torch.empty(n, dtype=torch.float32, device="cuda:0")
    B.check(B.fp16_to_fp32(master.data_ptr(), pm.data_ptr(), n), "fp16_to_fp32")
    mm = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    vm = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    for s in fx["fp16"]:
        g = dev16(s["g"])
        bc1 = float(np.array([s["bc1_bits"]], np.uint32).view(np.float32)[0])
        bc2 = float(np.array([s["bc2_bits"]], np.uint32).view(np.float32)[0])
        assert bc1 == host.bias_correction(hy["beta1"], s["step"]) and bc2 == host.bias_correction(hy["beta2"], s["step"])
        assert B.adamw_fp16(master.data_ptr(), pm.data_ptr(), g.data_ptr(), mm.data_ptr(), vm.data_ptr(), n, hy["lr"],
                            hy["beta1"], hy["beta2"], hy["eps"], hy["wd"], bc1, bc2) == B.OK
        torch.cuda.synchronize()
        assert bits(pm).tolist() == s["p_master"]
        assert bits(master).view(np.uint32).tolist() == s["master"]
    # without master copy, clip fused at step 2 through a plan
    p = dev16(p0)
    m = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    v = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    g = torch.zeros(n, dtype=torch.float16, device="cuda:0")
    plan = B.Plan([B.TensorDesc(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), None, n, B.DTYPE_F16, 0)], 2048)
    for s in fx["fp16"]:
        g.copy_(dev16(s["g"]))
        plan.grad_norm(0.05)
        norm, scale, _ = plan.norm_read()
        want_norm = float(np.array([s["norm_bits"]], np.uint32).view(np.float32)[0])
        assert abs(norm - want_norm) <= 1e-5 * want_norm
        sp = B.StepParams(hy["lr"], hy["beta1"], hy["beta2"], hy["eps"], hy["wd"],
                          host.bias_correction(hy["beta1"], s["step"]), host.bias_correction(hy["beta2"], s["step"]))
        if s["step"] == 2:
            # the stored step was clipped with the oracle's FP64-accumulated scale; the device's scale may differ
            # in the last bit, so feed the stored scale through the unfused route: scale on the host, then step
            want_scale = np.array([s["scale_bits"]], np.uint32).view(np.float32)[0]
            assert abs(scale - float(want_scale)) <= 2e-7 * float(want_scale)
            if scale == float(want_scale):
                plan.adamw(sp, B.CLIP_FUSED)
            else:
                # g' = f2h(h2f(g) * scale) with the stored scale (numpy's float16 conversion rounds to nearest
                # even, like the scale pass), then a plain step: what the fused step does with that scale
                scaled = (np.array(s["g"], np.uint16).view(np.float16).astype(np.float32) * want_scale).astype(np.float16)
                g.copy_(dev16(scaled.view(np.uint16)))
                plan.adamw(sp, B.CLIP_NONE)
        else:
            plan.adamw(sp, B.CLIP_NONE)
        torch.cuda.synchronize()
        assert bits(p).tolist() == s["p"] and bits(m).view(np.uint32).tolist() == s["m"]
        assert bits(v).view(np.uint32).tolist() == s["v"]
    plan.destroy()


def test_against_frozen_vectors_fp32(B, host, torch_gpu):
    """The FP32 operator on the inputs of tests/golden/adamw_regression.json (from the shared generator, seeds as
    in the fixture's script) against the two steps stored there."""
    import json
    import os
    torch = torch_gpu
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    fx = json.load(open(os.path.join(root, "tests", "golden", "adamw_regression.json")))
    n, hy = fx["n"], fx["hyper"]
    w = torch.empty(n, dtype=torch.float32, device="cuda:0")
    g32 = torch.empty(n, dtype=torch.float32, device="cuda:0")
    m32 = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    v32 = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    B.fill_f32(w.data_ptr(), n, 21, 1.0, 0.05)
    for s in fx["fp32"]:
        B.fill_f32(g32.data_ptr(), n, 30 + s["step"], 0.0, 1e-2)
        assert B.adamw_fp32(w.data_ptr(), g32.data_ptr(), m32.data_ptr(), v32.data_ptr(), n, hy["lr"], hy["beta1"],
                            hy["beta2"], hy["eps"], 0.0, host.bias_correction(hy["beta1"], s["step"]),
                            host.bias_correction(hy["beta2"], s["step"])) == B.OK
        torch.cuda.synchronize()
        assert bits(w).view(np.uint32).tolist() == s["w"] and bits(m32).view(np.uint32).tolist() == s["m"]
        assert bits(v32).view(np.uint32).tolist() == s["v"]


@pytest.mark.parametrize("eps,wd", [(1e-8, 0.01), (0.0, 0.0)])
@pytest.mark.parametrize("with_master", [False, True])
def test_every_half_gradient_against_special_moments(O, B, host, torch_gpu, eps, wd, with_master):
    """Every FP16 bit pattern as the gradient (zeros, subnormals, infinities, NaNs) crossed with FP32 moments
    and weights at the edges of the format: zero, negative zero, subnormal, the smallest and largest normal
    numbers, infinity, NaN, and a negative second moment.  IEEE division and square root, kept denormals and
    the final rounding to FP16 must give the oracle's bits; a NaN must meet a NaN (payloads are not compared)."""
    torch = torch_gpu
    f32 = np.float32
    m_set = np.array([0.0, -0.0, 1e-45, -3e-39, 1.17549435e-38, 1e-3, -7.5, 3.4e38, np.inf, -np.inf, np.nan], f32)
    v_set = np.array([0.0, 1e-45, 2e-39, 1.17549435e-38, 1e-20, 1e-6, 4.0, 3.4e38, np.inf, np.nan, -1e-6], f32)
    p_set = np.array([0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x2E66, 0xBC00, 0x7BFF, 0x7C00, 0x7E00], np.uint16)
    g_all = np.arange(65536, dtype=np.uint16)
    reps = len(m_set) * len(v_set)
    g_h = np.tile(g_all, reps)
    m_h = np.repeat(np.tile(m_set, len(v_set)), 65536).astype(f32)
    v_h = np.repeat(np.repeat(v_set, len(m_set)), 65536).astype(f32)
    n = g_h.size
    p_h = p_set[(np.arange(n) // 7) % len(p_set)].copy()
    w_h = O.h2f(p_h) if with_master else None

    def dev(a):
        t = torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).to("cuda:0")
        return t.view(torch.float16) if a.dtype == np.uint16 else t

    g_d, m_d, v_d, p_d = dev(g_h), dev(m_h), dev(v_h), dev(p_h)
    w_d = dev(w_h) if with_master else None
    bc1, bc2 = host.bias_correction(0.9, 3), host.bias_correction(0.999, 3)
    args = (1e-3, 0.9, 0.999, eps, wd, bc1, bc2)
    assert B.adamw_fp16(w_d.data_ptr() if with_master else None, p_d.data_ptr(), g_d.data_ptr(), m_d.data_ptr(),
                        v_d.data_ptr(), n, *args) == B.OK
    O.adamw_fp16(w_h, p_h, g_h, m_h, v_h, *args)
    torch.cuda.synchronize()

    def same(got, exp, what):
        if got.dtype == np.uint16:
            nan_g, nan_e = (got & 0x7FFF) > 0x7C00, (exp & 0x7FFF) > 0x7C00
            eq = got == exp
        else:
            nan_g, nan_e = np.isnan(got), np.isnan(exp)
            eq = got.view(np.uint32) == exp.view(np.uint32)
        bad = ~(eq | (nan_g & nan_e))
        assert not bad.any(), "%s: %d differ, first at %d: got %r expected %r" % (
            what, int(bad.sum()), int(np.argmax(bad)), got[np.argmax(bad)], exp[np.argmax(bad)])
        return int(nan_e.sum())

    nans = same(bits(p_d), p_h, "p") + same(bits(m_d), m_h, "m") + same(bits(v_d), v_h, "v")
    if with_master:
        same(bits(w_d), w_h, "master")
    assert nans > 0          # the grid does reach the non-finite cases


def test_fp32_update_on_random_bit_patterns(O, B, host, torch_gpu):
    """Four million elements whose weight, gradient and moments are uniformly random 32-bit patterns (every
    exponent, subnormals, infinities, NaNs, negative second moments): the FP32 update gives the oracle's bits
    wherever the oracle's result is a number, and a NaN wherever it is a NaN."""
    torch = torch_gpu
    n = 1 << 22
    rng = np.random.default_rng(20240607)
    host_arrays = [rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32) for _ in range(4)]
    w_h, g_h, m_h, v_h = host_arrays
    w_d, g_d, m_d, v_d = [torch.from_numpy(a.copy()).to("cuda:0") for a in host_arrays]
    bc1, bc2 = host.bias_correction(0.9, 7), host.bias_correction(0.999, 7)
    args = (1e-3, 0.9, 0.999, 1e-8, 0.01, bc1, bc2)
    assert B.adamw_fp32(w_d.data_ptr(), g_d.data_ptr(), m_d.data_ptr(), v_d.data_ptr(), n, *args) == B.OK
    O.adamw_fp32(w_h, g_h, m_h, v_h, *args)
    torch.cuda.synchronize()
    finite = 0
    for got, exp, what in ((bits(w_d), w_h, "w"), (bits(m_d), m_h, "m"), (bits(v_d), v_h, "v")):
        nan_g, nan_e = np.isnan(got), np.isnan(exp)
        bad = ~((got.view(np.uint32) == exp.view(np.uint32)) | (nan_g & nan_e))
        assert not bad.any(), "%s: %d differ, first at %d" % (what, int(bad.sum()), int(np.argmax(bad)))
        finite += int(np.isfinite(exp).sum())
    assert finite > n        # most results are numbers, not NaN


def test_clear_any_alignment_and_size(B, torch_gpu):
    """rlx_clear writes zeros to exactly the requested bytes: odd starts, odd lengths, and a range of more
    than 2 GiB; the bytes either side keep their pattern."""
    torch = torch_gpu
    span = 70_000
    for start, nbytes in [(0, span), (1, 1), (3, 13), (15, 17), (16, 4096), (5, 65_000), (129, 0), (31, 33)]:
        buf = torch.full((span,), 0xAB, dtype=torch.uint8, device="cuda:0")
        B.clear(buf.data_ptr() + start, nbytes)
        torch.cuda.synchronize()
        h = buf.cpu().numpy()
        exp = np.full(span, 0xAB, np.uint8)
        exp[start:start + nbytes] = 0
        assert np.array_equal(h, exp), (start, nbytes)
    big = torch.full(((1 << 31) + 4099,), 0x5A, dtype=torch.uint8, device="cuda:0")
    B.clear(big.data_ptr() + 3, (1 << 31) + 4090)
    torch.cuda.synchronize()
    assert int(big[:3].sum()) == 3 * 0x5A and int(big[-6:].sum()) == 6 * 0x5A
    assert int(big[3:-6].max()) == 0


@pytest.mark.parametrize("n,offset", [(1, 0), (3, 0), (4, 1), (4096, 0), (4097, 3), (1_000_003, 2)])
def test_scale_f32_equals_the_oracle(O, B, torch_gpu, n, offset):
    """The loss-gradient scale by 1/grad_accum_steps (include/training/trainer.h:96-99,261-263): one FP32
    multiply per element, any start alignment; the elements either side are untouched."""
    torch = torch_gpu
    buf = torch.empty(n + offset + 5, dtype=torch.float32, device="cuda:0")
    B.fill_f32(buf.data_ptr(), n + offset + 5, 77, 0.0, 3.0)
    torch.cuda.synchronize()
    h = bits(buf)
    scale = float(np.float32(1.0) / np.float32(3.0))
    B.scale_f32(buf.data_ptr() + 4 * offset, scale, n)
    O.scale_float(h[offset:offset + n], scale)
    torch.cuda.synchronize()
    assert np.array_equal(bits(buf).view(np.uint32), h.view(np.uint32))
