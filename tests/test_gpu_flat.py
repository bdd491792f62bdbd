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
