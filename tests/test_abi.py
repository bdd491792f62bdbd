"""CPU-only checks of the boundary: the shared library loads, exports every symbol that
include/rlx_adamw.h declares, and rejects bad arguments before touching a device."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "rlx_adamw.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rlx_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(B):
    lib = B.load()
    names = declared_symbols()
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), name + " is declared in the header but not exported"
    assert sorted(B.SIGNATURES) == names, "binding and header disagree"


def test_header_is_plain_c(tmp_path):
    """The header compiles as C99 with no HIP or torch headers in reach."""
    src = tmp_path / "t.c"
    src.write_text('#include "rlx_adamw.h"\nint main(void){rlx_step_params p; (void)p; return sizeof(rlx_tensor_desc) == 56 ? 0 : 1;}\n')
    exe = tmp_path / "t"
    assert os.system("gcc -std=c99 -Wall -Werror -I%s/include -o %s %s" % (ROOT, exe, src)) == 0
    assert os.system(str(exe)) == 0


def test_struct_layouts_match(B):
    assert C.sizeof(B.TensorDesc) == 56 and C.sizeof(B.StepParams) == 28


def test_version_and_status_strings(B):
    lib = B.load()
    assert lib.rlx_version() >= 100
    assert lib.rlx_status_string(B.OK) == b"ok"
    for st in range(1, B.ERR_WRONG_DEVICE + 1):
        assert lib.rlx_status_string(st) not in (b"ok", b"unknown status")
    assert lib.rlx_status_string(99) == b"unknown status"


def test_argument_checks_need_no_device(B):
    hyper = (1e-3, 0.9, 0.999, 1e-8, 0.01, 0.1, 0.001)
    # n <= 0 is a silent no-op (src/kernels/adamw.cu:49,99)
    assert B.adamw_fp16(None, None, None, None, None, 0, *hyper) == B.OK
    assert B.adamw_fp32(None, None, None, None, -1, *hyper) == B.OK
    assert B.fp16_to_fp32(None, None, 0) == B.OK
    # null pointers, misalignment, bad hyper-parameters: rejected on the host
    assert B.adamw_fp16(None, None, None, None, None, 8, *hyper) == B.ERR_INVALID_ARG
    assert B.adamw_fp16(None, 0x1001, 0x1000, 0x1000, 0x1000, 8, *hyper) == B.ERR_MISALIGNED
    assert B.adamw_fp32(0x1000, 0x1000, 0x1002, 0x1000, 8, *hyper) == B.ERR_MISALIGNED
    assert B.adamw_fp16(None, 0x1000, 0x1000, 0x1000, 0x1000, 8, 1e-3, 0.9, 0.999, 1e-8, 0.01, 0.0, 0.001) \
        == B.ERR_BAD_HYPER
    assert B.adamw_fp32(0x1000, 0x1000, 0x1000, 0x1000, 8, float("inf"), 0.9, 0.999, 1e-8, 0.0, 0.1, 0.1) \
        == B.ERR_BAD_HYPER
    assert B.fp16_to_fp32(0x1000, None, 4) == B.ERR_INVALID_ARG
    lib = B.load()
    assert lib.rlx_clear(None, 0, None) == B.OK and lib.rlx_clear(None, -5, None) == B.OK
    assert lib.rlx_clear(None, 16, None) == B.ERR_INVALID_ARG
    assert lib.rlx_scale_f32(None, 0.5, 0, None) == B.OK
    assert lib.rlx_scale_f32(None, 0.5, 4, None) == B.ERR_INVALID_ARG
    assert lib.rlx_scale_f32(0x1002, 0.5, 4, None) == B.ERR_MISALIGNED


def test_plan_argument_checks(B):
    lib = B.load()
    h = C.c_void_p()
    d = B.TensorDesc(0x1000, 0x2000, 0x3000, 0x4000, None, 100, B.DTYPE_F16, 0)
    arr = (B.TensorDesc * 1)(d)
    assert lib.rlx_plan_create(None, 1, 0, C.byref(h)) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_create(arr, 0, 0, C.byref(h)) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_create(arr, 1, 3000, C.byref(h)) == B.ERR_INVALID_ARG        # not a power of two
    assert lib.rlx_plan_create(arr, 1, 256, C.byref(h)) == B.ERR_INVALID_ARG         # below 512
    for bad in (B.TensorDesc(0x1000, 0x2000, 0x3000, 0x4000, None, 0, B.DTYPE_F16, 0),       # n == 0
                B.TensorDesc(0x1000, None, 0x3000, 0x4000, None, 8, B.DTYPE_F16, 0),          # no gradient
                B.TensorDesc(None, 0x2000, 0x3000, 0x4000, None, 8, B.DTYPE_F16, 0),          # no parameter
                B.TensorDesc(0x1000, 0x2000, 0x3000, 0x4000, None, 8, 7, 0),                  # dtype
                B.TensorDesc(0x1000, 0x2000, 0x3000, 0x4000, None, 8, B.DTYPE_F16, 64),       # flags
                B.TensorDesc(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 8, B.DTYPE_F32, 0)):     # master on FP32
        assert lib.rlx_plan_create((B.TensorDesc * 1)(bad), 1, 0, C.byref(h)) == B.ERR_INVALID_ARG
    odd = B.TensorDesc(0x1001, 0x2000, 0x3000, 0x4000, None, 8, B.DTYPE_F16, 0)
    assert lib.rlx_plan_create((B.TensorDesc * 1)(odd), 1, 0, C.byref(h)) == B.ERR_MISALIGNED
    assert h.value is None
    assert lib.rlx_plan_destroy(None) == B.OK
    assert lib.rlx_plan_num_chunks(None) == -1
    assert lib.rlx_plan_grad_norm(None, 1.0, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_adamw(None, None, 0, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_adamw_dev(None, None, 0, None) == B.ERR_INVALID_ARG
    sp = (B.StepParams * 1)(B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.0, 0.1, 0.001))
    assert lib.rlx_plan_schedule_upload(None, sp, 1, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_adamw_scheduled(None, 0, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_schedule_position(None, None, None, None) == B.ERR_INVALID_ARG
    over = C.c_int64(-1)
    assert lib.rlx_plan_schedule_overrun(None, C.byref(over), None) == B.ERR_INVALID_ARG and over.value == -1
    # the entry point that allocates nothing checks its arguments before it touches a device
    assert B.grad_norm_static(0x1000, -1, None, 0, 1.0, 0x2000) == B.ERR_INVALID_ARG
    assert B.grad_norm_static(None, 8, None, 0, 1.0, 0x2000) == B.ERR_INVALID_ARG
    assert B.grad_norm_static(0x1000, 8, None, 0, 1.0, None) == B.ERR_INVALID_ARG
    assert B.grad_norm_static(0x1001, 8, None, 0, 1.0, 0x2000) == B.ERR_MISALIGNED
    assert B.grad_norm_static(0x1000, 8, 0x3002, 8, 1.0, 0x2000) == B.ERR_MISALIGNED
    assert B.grad_norm_static(0x1000, 8, None, 0, 1.0, 0x2004) == B.ERR_MISALIGNED
    assert B.grad_norm_static(0x1000, 8, None, 0, 1.0, 0x2000, chunk_elems=1000) == B.ERR_INVALID_ARG
    assert B.grad_norm_static(0x1000, (1 << 18) * 512 + 1, None, 0, 1.0, 0x2000, chunk_elems=512) == B.ERR_TOO_LARGE


def test_tuning_keys(B):
    assert B.get_tuning("update_variant") == 0
    B.set_tuning("update_variant", 2)
    assert B.get_tuning("update_variant") == 2
    B.set_tuning("update_variant", 0)
    with pytest.raises(B.RlxError):
        B.set_tuning("update_variant", 99)
    with pytest.raises(B.RlxError):
        B.set_tuning("no_such_key", 1)
    assert B.get_tuning("no_such_key") == -1
    assert B.get_tuning("norm_fused") == 2 and B.get_tuning("norm_pack") == 3        # the shipped choices
    assert B.get_tuning("norm_keep_mb") == 0 and B.get_tuning("update_reverse") == 0
    for key, top in (("norm_pack", 3), ("convert_variant", 3), ("final_batch", 40), ("norm_fused", 1), ("norm_keep_mb", 4096),
                     ("update_reverse", 1)):
        default = B.get_tuning(key)
        B.set_tuning(key, top)
        assert B.get_tuning(key) == top
        B.set_tuning(key, default)
    with pytest.raises(B.RlxError):
        B.set_tuning("convert_variant", 4)
    with pytest.raises(B.RlxError):
        B.set_tuning("norm_fused", 3)
    with pytest.raises(B.RlxError):
        B.set_tuning("norm_keep_mb", 4097)
    # every update variant has a kernel name; the default names the shipped tile shape
    names = [B.update_variant_name(v) for v in range(18)]
    assert all(names) and len(set(names)) == 18 and B.update_variant_name(18) == ""
    assert names[0].startswith("adamw_tile_kernel<2,128,1,") and B.update_variant_name() == names[0]
    assert "persistent" in names[11] and "chunk" in names[12]


def test_layouts(L):
    """Tensor lists of the workloads (shapes of include/model/config.h:6-12; pool order of
    include/training/optimizer.h:30-32)."""
    s = L.qwen3_tensor_list(L.QWEN3_0_6B)
    assert len(s) == 310 and L.total_elements(s) == 596_049_920
    assert sum(t.n for t in s if t.row_len) == 595_984_384            # the FP16 pool of the reference
    assert [t.name for t in s[:7]] == ["layers.0." + k for k in
                                      ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")]
    assert s[196].name == "embed_tokens" and s[196].n == 151936 * 1024 and s[-1].name == "final_norm"
    ref = L.qwen3_tensor_list(L.QWEN3_0_6B, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
    assert sum(t.n for t in ref if t.dtype == L.DTYPE_F32) == 65_536
    assert all(t.flags & L.NO_DECAY for t in ref if t.dtype == L.DTYPE_F32 or t.name == "embed_tokens")
    assert not any(t.flags for t in ref if "proj" in t.name)
    big = L.qwen3_tensor_list(L.QWEN3_8B)
    assert len(big) == 399 and L.total_elements(big) == 8_190_427_136 + 308_224
    r = L.ragged_tensor_list()
    assert len(r) == 4096 and r == L.ragged_tensor_list()
    small = sum(1 for t in r if t.n in (128, 1024))
    assert 0.55 < small / 4096 < 0.65 and min(t.n for t in r) == 128 and max(t.n for t in r) <= 65536
    assert any(t.n % 8 for t in r)


def test_host_bias_correction_matches_oracle(host, O):
    for beta in (0.9, 0.999, 0.5):
        for t in (1, 2, 99, 100, 1000):
            assert host.bias_correction(beta, t) == O.bias_correction(beta, t)


def test_plan_create_without_a_device_reports_an_error(B):
    """Valid descriptors on a machine without a GPU: a status and a message, no crash.  (On a machine with
    a GPU the plan is only a table of addresses: it is created and destroyed without touching them.)"""
    lib = B.load()
    h = C.c_void_p()
    d = B.TensorDesc(0x10000, 0x20000, 0x30000, 0x40000, None, 5000, B.DTYPE_F16, 0)
    st = lib.rlx_plan_create((B.TensorDesc * 1)(d), 1, 0, C.byref(h))
    if st == B.OK:
        assert lib.rlx_plan_num_chunks(h) == 10 and lib.rlx_plan_num_elements(h) == 5000
        assert lib.rlx_plan_chunk_elems(h) == 512
        assert lib.rlx_plan_destroy(h) == B.OK
    else:
        assert st in (B.ERR_HIP, B.ERR_NO_DEVICE) and h.value is None
        assert lib.rlx_last_hip_error() != b""


def test_plan_layout_on_the_host(B, L):
    """Chunk size rule and chunk counts, computed without a device (include/rlx_adamw.h: rlx_plan_layout)."""
    def descs(sizes, dtype=None):
        out, at = [], 0x100000
        for n in sizes:
            out.append(B.TensorDesc(at, at + (1 << 40), at + (2 << 40), at + (3 << 40), None, n,
                                    B.DTYPE_F16 if dtype is None else dtype, 0))
            at += (n * 4 + 255) // 256 * 256
        return out
    # the automatic chunk follows the mean tensor size: 8192 from 32 Ki elements, 2048 from 8 Ki, else 512
    assert B.plan_layout(descs([32768]))[0] == 8192
    assert B.plan_layout(descs([32767]))[0] == 2048
    assert B.plan_layout(descs([8192]))[0] == 2048
    assert B.plan_layout(descs([8191]))[0] == 512
    assert B.plan_layout(descs([1]))[:2] == (512, 1)
    assert B.plan_layout(descs([100000, 128]))[0] == 8192          # mean 50,064
    # chunk count = sum of per-tensor ceilings; a tensor never shares a chunk with its neighbour
    sizes = [1, 511, 512, 513, 70000]
    for chunk in (512, 1024, 8192, 1 << 24):
        ce, nc, ne = B.plan_layout(descs(sizes), chunk)
        assert ce == chunk and ne == sum(sizes) and nc == sum(-(-n // chunk) for n in sizes)
    # the workloads of the benchmark
    q = L.qwen3_tensor_list(L.QWEN3_0_6B)
    assert B.plan_layout(descs([t.n for t in q])) == (8192, 72865, 596_049_920)
    r = L.ragged_tensor_list()
    ce, nc, ne = B.plan_layout(descs([t.n for t in r]))
    assert ce == 512 and ne == L.total_elements(r) and nc == sum(-(-t.n // 512) for t in r)
    big = L.qwen3_tensor_list(L.QWEN3_8B)
    ce, nc, ne = B.plan_layout(descs([t.n for t in big]))       # billions of elements: larger chunks, ~2^18 of them
    assert ce == 32768 and nc == sum(-(-t.n // 32768) for t in big) and nc <= (1 << 18)
    assert B.plan_layout(descs([t.n for t in big]), 8192)[1] == 999_953
    # same argument checks as rlx_plan_create
    lib = B.load()
    arr = (B.TensorDesc * 1)(*descs([5000]))
    assert lib.rlx_plan_layout(arr, 1, 3000, None, None, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_layout(arr, 1, 256, None, None, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_layout(arr, 1, 1 << 25, None, None, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_layout(None, 1, 0, None, None, None) == B.ERR_INVALID_ARG
    assert lib.rlx_plan_layout(arr, 1, 0, None, None, None) == B.OK
    huge = (B.TensorDesc * 1)(B.TensorDesc(0x1000, 0x2000, 0x3000, 0x4000, None, 1 << 41, B.DTYPE_F16, 0))
    assert lib.rlx_plan_layout(huge, 1, 512, None, None, None) == B.ERR_TOO_LARGE
