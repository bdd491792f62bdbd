"""Helpers shared by the GPU parity tests."""
import numpy as np

HYPER = dict(lr=1e-5, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)   # defaults of trainer.h:36-43


def bits(t):
    """torch tensor -> numpy (uint16 bit patterns for FP16)."""
    import torch
    if t.dtype == torch.float16:
        return t.detach().cpu().view(torch.int16).numpy().view(np.uint16).copy()
    return t.detach().cpu().numpy().copy()


def half_ulp_diff(a_bits, b_bits):
    """Distance in FP16 units of least precision between two bit-pattern arrays (finite values)."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def rel_err(a, b):
    a = a.astype(np.float64)
    b = b.astype(np.float64)
    den = np.maximum(np.abs(b), np.finfo(np.float32).tiny)
    return np.abs(a - b) / den


def check_state(got_p, got_m, got_v, exp_p, exp_m, exp_v, what=""):
    """The tolerances of the path: FP32 moments 1e-6 relative, FP16 weights 1 ulp.
    Returns how many values were not bit-identical (for reporting)."""
    assert rel_err(got_m, exp_m).max() <= 1e-6, what + " m"
    assert rel_err(got_v, exp_v).max() <= 1e-6, what + " v"
    if got_p.dtype == np.uint16:
        assert half_ulp_diff(got_p, exp_p).max() <= 1, what + " p"
    else:
        assert rel_err(got_p, exp_p).max() <= 1e-6, what + " p"
    return int((got_p != exp_p).sum() + (got_m.view(np.uint32) != exp_m.view(np.uint32)).sum()
               + (got_v.view(np.uint32) != exp_v.view(np.uint32)).sum())


def read_device(ptr, nbytes):
    """Bytes at a raw device address, copied with the HIP runtime that the process already has loaded."""
    import ctypes as C
    path = next(line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line)
    hip = C.CDLL(path)
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    hip.hipMemcpy.restype = C.c_int
    buf = np.empty(nbytes, np.uint8)
    rc = hip.hipMemcpy(buf.ctypes.data, ptr, nbytes, 2)          # 2 = device to host; waits for earlier work
    assert rc == 0, "hipMemcpy failed: %d" % rc
    return buf
