"""ctypes loader for the CPU oracle (liborc_adamw.so).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the bench's cpu_baseline leg import this module; the
product package never does.  All functions take numpy arrays (uint16 for FP16 bits,
float32, float64) and work in place where the reference does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liborc_adamw.so")

FILL_ABS = 1


def build(force=False):
    """Compile the oracle with gcc through its Makefile."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def _load():
    if not os.path.exists(_SO):
        build()
    lib = C.CDLL(_SO)
    f, i64, u16p, f32p, f64p, vp, u64, u32, i32 = (
        C.c_float, C.c_int64, C.POINTER(C.c_uint16), C.POINTER(C.c_float), C.POINTER(C.c_double),
        C.c_void_p, C.c_uint64, C.c_uint32, C.c_int)
    hyper = [f] * 7
    sig = {
        "orc_h2f": ([C.c_uint16], f),
        "orc_f2h": ([f], C.c_uint16),
        "orc_h2f_array": ([vp, vp, i64], None),
        "orc_f2h_array": ([vp, vp, i64], None),
        "orc_fp16_to_fp32": ([vp, vp, i64], None),
        "orc_bias_correction": ([f, i32], f),
        "orc_adamw_fp16": ([vp, vp, vp, vp, vp, i64] + hyper, None),
        "orc_adamw_fp16_clip": ([vp, vp, vp, vp, vp, i64] + hyper + [f, i32], None),
        "orc_adamw_fp32": ([vp, vp, vp, vp, i64] + hyper, None),
        "orc_adamw_fp32_clip": ([vp, vp, vp, vp, i64] + hyper + [f, i32], None),
        "orc_optimizer_step": ([vp, vp, vp, vp, vp, i64, i64, vp, vp, vp, vp, i64, f, f, f, f, f,
                                C.POINTER(i32)], None),
        "orc_sum_sq_half": ([vp, i64], C.c_double),
        "orc_sum_sq_float": ([vp, i64], C.c_double),
        "orc_scale_half": ([vp, f, i64], None),
        "orc_scale_float": ([vp, f, i64], None),
        "orc_clip_scale": ([f, f, f32p], f),
        "orc_clip_grad_norm": ([vp, i64, vp, i64, f, f32p], f),
        "orc_sumsq_mirror_partials": ([vp, i32, i64, i32, vp], i64),
        "orc_sumsq_mirror_final": ([vp, i64], C.c_double),
        "orc_sumsq_mirror_groups": ([vp, i64, vp], i64),
        "orc_sumsq_mirror_total": ([vp, i64, i32], C.c_double),
        "orc_fill_f16": ([vp, i64, u64, i64, f, f, u32, i64, u32], None),
        "orc_fill_f32": ([vp, i64, u64, i64, f, f, u32, i64, u32], None),
        "orc_step_fp16_threaded": ([vp, vp, vp, vp, vp, i64] + hyper + [f, i32], f),
        "orc_step_list_fp16_threaded": ([i64, vp, vp, vp, vp, vp] + hyper + [f, i32], f),
        "orc_update_per_tensor_fp16_threaded": ([i64, vp, vp, vp, vp, vp] + hyper + [i32], None),
    }
    for name, (args, res) in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    del u16p, f64p, u32
    return lib


lib = _load()


def _p(a, dtype):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.dtype == dtype and a.flags.c_contiguous, (a.dtype, dtype)
    return a.ctypes.data


U16, F32, F64 = np.dtype(np.uint16), np.dtype(np.float32), np.dtype(np.float64)


def h2f(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.orc_h2f_array(_p(out, F32), _p(h, U16), h.size)
    return out


def f2h(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.orc_f2h_array(_p(out, U16), _p(x, F32), x.size)
    return out


def bias_correction(beta, step):
    return float(lib.orc_bias_correction(beta, step))


def adamw_fp16(master, model, grad, m, v, lr, beta1, beta2, eps, wd, bc1, bc2, clip_scale=None):
    n = model.size
    if clip_scale is None:
        lib.orc_adamw_fp16(_p(master, F32), _p(model, U16), _p(grad, U16), _p(m, F32), _p(v, F32), n,
                           lr, beta1, beta2, eps, wd, bc1, bc2)
    else:
        lib.orc_adamw_fp16_clip(_p(master, F32), _p(model, U16), _p(grad, U16), _p(m, F32), _p(v, F32), n,
                                lr, beta1, beta2, eps, wd, bc1, bc2, clip_scale, 1)


def adamw_fp32(w, grad, m, v, lr, beta1, beta2, eps, wd, bc1, bc2, clip_scale=None):
    n = w.size
    if clip_scale is None:
        lib.orc_adamw_fp32(_p(w, F32), _p(grad, F32), _p(m, F32), _p(v, F32), n,
                           lr, beta1, beta2, eps, wd, bc1, bc2)
    else:
        lib.orc_adamw_fp32_clip(_p(w, F32), _p(grad, F32), _p(m, F32), _p(v, F32), n,
                                lr, beta1, beta2, eps, wd, bc1, bc2, clip_scale, 1)


def optimizer_step(master, pool16, g16, m16, v16, proj_n, pool32, g32, m32, v32,
                   lr, beta1, beta2, eps, wd, step):
    """Returns the incremented step counter."""
    st = C.c_int(step)
    lib.orc_optimizer_step(_p(master, F32), _p(pool16, U16), _p(g16, U16), _p(m16, F32), _p(v16, F32),
                           pool16.size, proj_n, _p(pool32, F32), _p(g32, F32), _p(m32, F32), _p(v32, F32),
                           pool32.size, lr, beta1, beta2, eps, wd, C.byref(st))
    return st.value


def sum_sq_half(g):
    return float(lib.orc_sum_sq_half(_p(g, U16), g.size))


def sum_sq_float(g):
    return float(lib.orc_sum_sq_float(_p(g, F32), g.size))


def scale_half(g, scale):
    lib.orc_scale_half(_p(g, U16), scale, g.size)


def scale_float(g, scale):
    lib.orc_scale_float(_p(g, F32), scale, g.size)


def clip_scale(sum_sq, max_norm):
    """(scale, norm) of the clip rule for a given FP32 sum of squares."""
    norm = C.c_float(0)
    s = lib.orc_clip_scale(sum_sq, max_norm, C.byref(norm))
    return float(s), float(norm.value)


def clip_grad_norm(half_pool, float_pool, max_norm):
    """In place.  Returns (pre-clip norm, applied scale)."""
    sc = C.c_float(0)
    n16 = 0 if half_pool is None else half_pool.size
    n32 = 0 if float_pool is None else float_pool.size
    norm = lib.orc_clip_grad_norm(_p(half_pool, U16), n16, _p(float_pool, F32), n32, max_norm, C.byref(sc))
    return float(norm), float(sc.value)


def sumsq_mirror_final(values):
    """The fixed-order FP64 sum of the last step of the device's norm (over chunk partials, or over group
    partials for 512-element chunks)."""
    allp = np.ascontiguousarray(values, dtype=np.float64)
    return float(lib.orc_sumsq_mirror_final(_p(allp, F64), allp.size))


def sumsq_mirror_groups(partials):
    """Group partials of a plan with 512-element chunks: 16 consecutive chunk partials added in order."""
    allp = np.ascontiguousarray(partials, dtype=np.float64)
    out = np.empty(max((allp.size + 15) // 16, 1), np.float64)
    k = lib.orc_sumsq_mirror_groups(_p(allp, F64), allp.size, _p(out, F64))
    return out[:k]


def sumsq_mirror_total(partials, chunk):
    """The device's sum of squares from its per-chunk partials, for a plan with chunks of `chunk` elements."""
    allp = np.ascontiguousarray(partials, dtype=np.float64)
    return float(lib.orc_sumsq_mirror_total(_p(allp, F64), allp.size, chunk))


def sumsq_mirror(grads, chunk):
    """Sum of squares of a list of gradient arrays in the device's reduction order."""
    parts = []
    for g in grads:
        is_f32 = g.dtype == F32
        k = (g.size + chunk - 1) // chunk
        buf = np.empty(max(k, 1), np.float64)
        got = lib.orc_sumsq_mirror_partials(_p(g, F32 if is_f32 else U16), int(is_f32), g.size, chunk,
                                            _p(buf, F64))
        assert got == k
        parts.append(buf[:k])
    allp = np.ascontiguousarray(np.concatenate(parts)) if parts else np.zeros(0, np.float64)
    return float(lib.orc_sumsq_mirror_total(_p(allp, F64), allp.size, chunk)), allp


def fill_f16(n, seed, mean, std, first=0, flags=0, row_len=0, zero_rows_below=0):
    out = np.empty(n, np.uint16)
    lib.orc_fill_f16(_p(out, U16), n, seed, first, mean, std, flags, row_len, zero_rows_below)
    return out


def fill_f32(n, seed, mean, std, first=0, flags=0, row_len=0, zero_rows_below=0):
    out = np.empty(n, np.float32)
    lib.orc_fill_f32(_p(out, F32), n, seed, first, mean, std, flags, row_len, zero_rows_below)
    return out


def step_fp16_threaded(master, model, grad, m, v, lr, beta1, beta2, eps, wd, bc1, bc2, max_norm, threads):
    return float(lib.orc_step_fp16_threaded(_p(master, F32), _p(model, U16), _p(grad, U16), _p(m, F32),
                                            _p(v, F32), model.size, lr, beta1, beta2, eps, wd, bc1, bc2,
                                            max_norm, threads))


def list_pointers(p_pool, g_pool, m_pool, v_pool, off_pg, off_state, counts):
    """The pointer arrays of a tensor list inside four pools (FP16 weights and gradients share the offsets off_pg,
    FP32 moments the offsets off_state; counts[i] elements each), built once for repeated calls.  The pools must
    stay alive and in place while the result is used."""
    k = len(counts)
    ptr = C.c_void_p * k
    cnt = (C.c_int64 * k)(*[int(c) for c in counts])
    model = ptr(*[_p(p_pool, U16) + 2 * int(o) for o in off_pg])
    grad = ptr(*[_p(g_pool, U16) + 2 * int(o) for o in off_pg])
    m = ptr(*[_p(m_pool, F32) + 4 * int(o) for o in off_state])
    v = ptr(*[_p(v_pool, F32) + 4 * int(o) for o in off_state])
    return k, model, grad, m, v, cnt


def step_list_fp16_threaded(p_pool, g_pool, m_pool, v_pool, off_pg, off_state, counts, lr, beta1, beta2, eps, wd,
                            bc1, bc2, max_norm, threads, pointers=None):
    """Norm (if max_norm > 0) + clip + update of a LIST of FP16 tensors that live inside four pools, with the
    concatenated index space split over `threads` host threads.  In place.  Returns the pre-clip norm.
    `pointers`: the result of list_pointers for these pools (saves building it on every call)."""
    k, model, grad, m, v, cnt = pointers or list_pointers(p_pool, g_pool, m_pool, v_pool, off_pg, off_state, counts)
    return float(lib.orc_step_list_fp16_threaded(k, model, grad, m, v, cnt, lr, beta1, beta2, eps, wd, bc1, bc2,
                                                 max_norm, threads))


def update_per_tensor_fp16_threaded(p_pool, g_pool, m_pool, v_pool, off_pg, off_state, counts, lr, beta1, beta2, eps,
                                    wd, bc1, bc2, threads, pointers=None):
    """The same update as a loop over the tensors, each split over the threads by itself."""
    k, model, grad, m, v, cnt = pointers or list_pointers(p_pool, g_pool, m_pool, v_pool, off_pg, off_state, counts)
    lib.orc_update_per_tensor_fp16_threaded(k, model, grad, m, v, cnt, lr, beta1, beta2, eps, wd, bc1, bc2, threads)
