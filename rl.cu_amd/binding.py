"""ctypes binding of librlx_adamw.so (the C ABI in include/rlx_adamw.h).

Pointers are plain integers (for torch tensors: tensor.data_ptr()); streams are
hipStream_t handles as integers (torch.cuda.current_stream().cuda_stream), 0 = default.
There is no CPU fallback: if the library is missing, loading raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "librlx_adamw.so")

(OK, ERR_INVALID_ARG, ERR_MISALIGNED, ERR_BAD_HYPER, ERR_HIP, ERR_NO_DEVICE, ERR_TOO_LARGE, ERR_NO_MEMORY,
 ERR_WRONG_DEVICE) = range(9)
DTYPE_F16, DTYPE_F32 = 0, 1
TENSOR_NO_DECAY, TENSOR_GRAD_ONLY, TENSOR_FROZEN = 1, 2, 4
CLIP_NONE, CLIP_FUSED, STEP_ZERO_GRADS = 0, 1, 2
FILL_ABS = 1


class RlxError(RuntimeError):
    def __init__(self, status, where, detail=""):
        self.status = status
        super().__init__("%s: status %d (%s)%s" % (where, status, _status_string(status), detail))


class TensorDesc(C.Structure):
    _fields_ = [("param", C.c_void_p), ("grad", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p),
                ("master", C.c_void_p), ("n", C.c_int64), ("dtype", C.c_int32), ("flags", C.c_uint32)]


class StepParams(C.Structure):
    _fields_ = [("lr", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("eps", C.c_float),
                ("weight_decay", C.c_float), ("bias_correction1", C.c_float), ("bias_correction2", C.c_float)]


_F, _I64, _VP, _U64, _U32, _INT = C.c_float, C.c_int64, C.c_void_p, C.c_uint64, C.c_uint32, C.c_int
_HYPER = [_F] * 7

# name -> (argtypes, restype): every symbol that include/rlx_adamw.h declares
SIGNATURES = {
    "rlx_status_string": ([_INT], C.c_char_p),
    "rlx_last_hip_error": ([], C.c_char_p),
    "rlx_version": ([], _INT),
    "rlx_adamw_fp16": ([_VP, _VP, _VP, _VP, _VP, _I64] + _HYPER + [_VP], _INT),
    "rlx_adamw_fp32": ([_VP, _VP, _VP, _VP, _I64] + _HYPER + [_VP], _INT),
    "rlx_fp16_to_fp32": ([_VP, _VP, _I64, _VP], _INT),
    "rlx_clear": ([_VP, _I64, _VP], _INT),
    "rlx_scale_f32": ([_VP, _F, _I64, _VP], _INT),
    "rlx_plan_create": ([C.POINTER(TensorDesc), _I64, _I64, C.POINTER(_VP)], _INT),
    "rlx_plan_layout": ([C.POINTER(TensorDesc), _I64, _I64, C.POINTER(_I64), C.POINTER(_I64), C.POINTER(_I64)], _INT),
    "rlx_plan_destroy": ([_VP], _INT),
    "rlx_plan_num_chunks": ([_VP], _I64),
    "rlx_plan_num_elements": ([_VP], _I64),
    "rlx_plan_chunk_elems": ([_VP], _I64),
    "rlx_plan_grad_norm": ([_VP, _F, _VP], _INT),
    "rlx_grad_norm_static": ([_VP, _I64, _VP, _I64, _I64, _F, _VP, _VP], _INT),
    "rlx_plan_norm_read": ([_VP, C.POINTER(_F), C.POINTER(_F), C.POINTER(C.c_double), _VP], _INT),
    "rlx_plan_norm_device_ptr": ([_VP], _VP),
    "rlx_plan_partials_device_ptr": ([_VP], _VP),
    "rlx_plan_scale_grads": ([_VP, _VP], _INT),
    "rlx_plan_adamw": ([_VP, C.POINTER(StepParams), _INT, _VP], _INT),
    "rlx_plan_adamw_dev": ([_VP, _VP, _INT, _VP], _INT),
    "rlx_plan_schedule_upload": ([_VP, C.POINTER(StepParams), _I64, _VP], _INT),
    "rlx_plan_adamw_scheduled": ([_VP, _INT, _VP], _INT),
    "rlx_plan_schedule_position": ([_VP, C.POINTER(_I64), C.POINTER(_I64), _VP], _INT),
    "rlx_plan_schedule_overrun": ([_VP, C.POINTER(_I64), _VP], _INT),
    "rlx_update_variant_name": ([_I64], C.c_char_p),
    "rlx_set_tuning": ([C.c_char_p, _I64], _INT),
    "rlx_get_tuning": ([C.c_char_p], _I64),
    "rlx_fill_f16": ([_VP, _I64, _U64, _I64, _F, _F, _U32, _I64, _U32, _VP], _INT),
    "rlx_fill_f32": ([_VP, _I64, _U64, _I64, _F, _F, _U32, _I64, _U32, _VP], _INT),
}

_lib = None


ABI_VERSION = 109        # rlx_version() of the library this binding was written against


def load():
    """Loads the built library; there is no CPU fallback of any kind.
    Missing library: it is compiled first, and loading raises if that fails.
    Library whose source stamp (the hash of its sources that this package's build leaves next to it) differs from
    the tree: it is compiled again; if that cannot be done (no hipcc on this machine) the existing library is
    loaded with a warning.
    Library without a stamp (built with the documented hipcc line or by CMake): loaded as it is.
    In every case the loaded library must report the ABI version that this binding was written against."""
    global _lib
    if _lib is not None:
        return _lib
    from . import build as _build
    if not os.path.exists(LIB_PATH):
        try:
            _build.build_library()
        except Exception as exc:
            raise RuntimeError("librlx_adamw.so is not built (%s) and building it failed: %s" % (LIB_PATH, exc))
    elif _build.is_stale():
        try:
            _build.build_library()
        except Exception as exc:
            import warnings
            warnings.warn("librlx_adamw.so was built from other sources than the tree holds and could not be rebuilt "
                          "(%s); loading it as it is" % exc)
    try:
        # torch, when present, brings its own HIP runtime: load it first so that this library
        # binds to the same runtime instance as the tensors it is handed.
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    for name, (args, res) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    if lib.rlx_version() != ABI_VERSION:
        raise RuntimeError("librlx_adamw.so reports ABI version %d, this binding expects %d: rebuild the library "
                           "(python rl.cu_amd/build.py)" % (lib.rlx_version(), ABI_VERSION))
    _lib = lib
    return lib


def _status_string(status):
    try:
        return load().rlx_status_string(status).decode()
    except Exception:  # pragma: no cover
        return "?"


def check(status, where):
    if status != OK:
        detail = ""
        if status == ERR_HIP:
            detail = " " + load().rlx_last_hip_error().decode()
        raise RlxError(status, where, detail)


def set_tuning(key, value):
    check(load().rlx_set_tuning(key.encode(), int(value)), "rlx_set_tuning(%s)" % key)


def get_tuning(key):
    return int(load().rlx_get_tuning(key.encode()))


def update_variant_name(variant=None):
    """Kernel instantiation behind an update_variant number (default: the active one)."""
    v = get_tuning("update_variant") if variant is None else variant
    return load().rlx_update_variant_name(v).decode()


def adamw_fp16(master_w, model_w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay, bc1, bc2, stream=0):
    """launch_adamw_fp16 (include/kernels/adamw.cuh:24-39); returns the status."""
    return load().rlx_adamw_fp16(master_w, model_w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay,
                                 bc1, bc2, stream)


def adamw_fp32(w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay, bc1, bc2, stream=0):
    """launch_adamw_fp32 (include/kernels/adamw.cuh:43-57); returns the status."""
    return load().rlx_adamw_fp32(w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay, bc1, bc2, stream)


def fp16_to_fp32(dst, src, n, stream=0):
    return load().rlx_fp16_to_fp32(dst, src, n, stream)


def fill_f16(dst, n, seed, mean, std, first=0, flags=0, row_len=0, zero_rows_below=0, stream=0):
    check(load().rlx_fill_f16(dst, n, seed, first, mean, std, flags, row_len, zero_rows_below, stream),
          "rlx_fill_f16")


def fill_f32(dst, n, seed, mean, std, first=0, flags=0, row_len=0, zero_rows_below=0, stream=0):
    check(load().rlx_fill_f32(dst, n, seed, first, mean, std, flags, row_len, zero_rows_below, stream),
          "rlx_fill_f32")


def clear(dst, nbytes, stream=0):
    check(load().rlx_clear(dst, nbytes, stream), "rlx_clear")


def scale_f32(x, scale, n, stream=0):
    check(load().rlx_scale_f32(x, scale, n, stream), "rlx_scale_f32")


def grad_norm_static(half_grads, n_half, float_grads, n_float, max_norm, result_dev, chunk_elems=0, stream=0):
    """Norm and clip scale of two flat gradient buffers into 16 bytes at result_dev; allocates nothing.
    Returns the status."""
    return load().rlx_grad_norm_static(half_grads, n_half, float_grads, n_float, chunk_elems, max_norm, result_dev,
                                       stream)


def plan_layout(descs, chunk_elems=0):
    """(chunk_elems, num_chunks, num_elements) that a plan over `descs` would have; host only."""
    arr = (TensorDesc * len(descs))(*descs)
    ce, nc, ne = _I64(), _I64(), _I64()
    check(load().rlx_plan_layout(arr, len(descs), chunk_elems, C.byref(ce), C.byref(nc), C.byref(ne)),
          "rlx_plan_layout")
    return ce.value, nc.value, ne.value


class Plan:
    """Owner of one rlx_plan.  `descs` is a list of TensorDesc (pointers are borrowed)."""

    def __init__(self, descs, chunk_elems=0):
        self._h = None
        arr = (TensorDesc * len(descs))(*descs)
        h = _VP()
        check(load().rlx_plan_create(arr, len(descs), chunk_elems, C.byref(h)), "rlx_plan_create")
        self._h = h
        self.count = len(descs)

    @property
    def num_chunks(self):
        return int(load().rlx_plan_num_chunks(self._h))

    @property
    def num_elements(self):
        return int(load().rlx_plan_num_elements(self._h))

    @property
    def chunk_elems(self):
        return int(load().rlx_plan_chunk_elems(self._h))

    @property
    def partials_ptr(self):
        return load().rlx_plan_partials_device_ptr(self._h)

    @property
    def norm_ptr(self):
        return load().rlx_plan_norm_device_ptr(self._h)

    def grad_norm(self, max_norm, stream=0):
        check(load().rlx_plan_grad_norm(self._h, max_norm, stream), "rlx_plan_grad_norm")

    def norm_read(self, stream=0):
        """Blocking.  Returns (norm, scale, sum_sq)."""
        n, s, q = _F(0), _F(0), C.c_double(0)
        check(load().rlx_plan_norm_read(self._h, C.byref(n), C.byref(s), C.byref(q), stream),
              "rlx_plan_norm_read")
        return float(n.value), float(s.value), float(q.value)

    def scale_grads(self, stream=0):
        check(load().rlx_plan_scale_grads(self._h, stream), "rlx_plan_scale_grads")

    def adamw(self, params, step_flags=CLIP_NONE, stream=0):
        check(load().rlx_plan_adamw(self._h, C.byref(params), step_flags, stream), "rlx_plan_adamw")

    def adamw_dev(self, dev_params_ptr, step_flags=CLIP_NONE, stream=0):
        check(load().rlx_plan_adamw_dev(self._h, dev_params_ptr, step_flags, stream), "rlx_plan_adamw_dev")

    def schedule_upload(self, steps, stream=0):
        """steps: list of StepParams for the coming scheduled steps (validated; blocking)."""
        arr = (StepParams * len(steps))(*steps)
        check(load().rlx_plan_schedule_upload(self._h, arr, len(steps), stream), "rlx_plan_schedule_upload")

    def adamw_scheduled(self, step_flags=CLIP_NONE, stream=0):
        check(load().rlx_plan_adamw_scheduled(self._h, step_flags, stream), "rlx_plan_adamw_scheduled")

    def schedule_position(self, stream=0):
        """Blocking.  Returns (scheduled steps taken since the upload, length of the table)."""
        taken, total = _I64(), _I64()
        check(load().rlx_plan_schedule_position(self._h, C.byref(taken), C.byref(total), stream),
              "rlx_plan_schedule_position")
        return taken.value, total.value

    def schedule_overrun(self, stream=0):
        """Blocking.  Scheduled updates since the upload that ran after the table had been used up."""
        over = _I64()
        check(load().rlx_plan_schedule_overrun(self._h, C.byref(over), stream), "rlx_plan_schedule_overrun")
        return over.value

    def destroy(self):
        if self._h is not None:
            h, self._h = self._h, None
            check(load().rlx_plan_destroy(h), "rlx_plan_destroy")

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
