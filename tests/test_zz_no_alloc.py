"""rlx_grad_norm_static, the entry point that allocates nothing, against rlx_plan_grad_norm over the same two
gradient buffers: the 16 result bytes must be identical, on two calls in a row, the second with a smaller input.
Runs last in the suite (file name), and must also pass alone in a fresh process."""
import numpy as np
import pytest

from util import read_device

pytestmark = pytest.mark.gpu


def plan_result(B, g16, n16, g32, n32, chunk, max_norm, stream):
    """{sum_sq, norm, scale} as 16 bytes from the plan-based entry point."""
    descs = []
    if n16:
        descs.append(B.TensorDesc(None, g16.data_ptr(), None, None, None, n16, B.DTYPE_F16, B.TENSOR_GRAD_ONLY))
    if n32:
        descs.append(B.TensorDesc(None, g32.data_ptr(), None, None, None, n32, B.DTYPE_F32, B.TENSOR_GRAD_ONLY))
    plan = B.Plan(descs, chunk)
    plan.grad_norm(max_norm, stream)
    out = read_device(plan.norm_ptr, 16).copy()
    chunk_used = plan.chunk_elems
    plan.destroy()
    return out, chunk_used


def test_static_norm_equals_plan_norm_twice_second_smaller(B, torch_gpu):
    torch = torch_gpu
    stream = torch.cuda.current_stream().cuda_stream
    n16_big, n32_big = 3_000_017, 70_003
    g16 = torch.empty(n16_big, dtype=torch.float16, device="cuda:0")
    g32 = torch.empty(n32_big, dtype=torch.float32, device="cuda:0")
    B.fill_f16(g16.data_ptr(), n16_big, 101, 0.0, 5e-3, stream=stream)
    B.fill_f32(g32.data_ptr(), n32_big, 102, 0.0, 2e-2, stream=stream)
    result = torch.zeros(2, dtype=torch.float64, device="cuda:0")      # 16 bytes, caller-owned output
    torch.cuda.synchronize()

    # first call on this device resolves the array's address; later calls must leave free memory unchanged
    assert B.grad_norm_static(g16.data_ptr(), 1024, g32.data_ptr(), 0, 1.0, result.data_ptr(), 0, stream) == B.OK
    torch.cuda.synchronize()

    # (n16, n32, chunk_elems, max_norm): large, then smaller inputs on the same scratch, then edge shapes
    cases = [(n16_big, n32_big, 0, 1.0), (40_961, 1_025, 0, 1.0), (n16_big, n32_big, 512, 1.0),
             (777, 0, 2048, 1e9), (0, 4_099, 8192, 0.01), (n16_big, n32_big, 65536, float("inf"))]
    results = torch.full((len(cases), 2), -1.0, dtype=torch.float64, device="cuda:0")   # one 16-byte output per call
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for k, (n16, n32, chunk, max_norm) in enumerate(cases):      # back to back on one stream, nothing in between
        st = B.grad_norm_static(g16.data_ptr(), n16, g32.data_ptr(), n32, max_norm, results[k].data_ptr(), chunk,
                                stream)
        assert st == B.OK, (st, n16, n32, chunk)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "rlx_grad_norm_static changed the free device memory"
    got = [read_device(results[k].data_ptr(), 16).copy() for k in range(len(cases))]

    for (n16, n32, chunk, max_norm), g in zip(cases, got):
        want, _ = plan_result(B, g16, n16, g32, n32, chunk, max_norm, stream)
        assert np.array_equal(g, want), ("static norm differs from the plan's", n16, n32, chunk,
                                         g.view(np.float64)[0], want.view(np.float64)[0])
        # and both against FP64 on the host (1e-5 relative, the path's tolerance for the norm)
        h16 = g16[:n16].cpu().numpy().astype(np.float64)
        h32 = g32[:n32].cpu().numpy().astype(np.float64)
        exact = float(np.sqrt((h16 * h16).sum() + (h32 * h32).sum()))
        norm, scale = g.view(np.float32)[2], g.view(np.float32)[3]
        assert abs(norm - exact) <= 1e-5 * exact, (norm, exact)
        want_scale = np.float32(max_norm) / (norm + np.float32(1e-6)) if norm > np.float32(max_norm) else np.float32(1.0)
        assert scale == want_scale


def test_static_norm_empty_input_and_limits(B, torch_gpu):
    torch = torch_gpu
    stream = torch.cuda.current_stream().cuda_stream
    g16 = torch.zeros(4096, dtype=torch.float16, device="cuda:0")
    result = torch.full((2,), -1.0, dtype=torch.float64, device="cuda:0")
    # nothing to add up: sum 0, norm 0, scale 1
    assert B.grad_norm_static(0, 0, 0, 0, 1.0, result.data_ptr(), 0, stream) == B.OK
    torch.cuda.synchronize()
    out = read_device(result.data_ptr(), 16)
    assert out.view(np.float64)[0] == 0.0 and out.view(np.float32)[2] == 0.0 and out.view(np.float32)[3] == 1.0
    # more chunks than the static array holds: refused before anything is launched (no memory is touched:
    # 2^18 chunks of 512 elements + 1 would need 134,217,729 elements; only the size is checked)
    too_many = (1 << 18) * 512 + 1
    assert B.grad_norm_static(g16.data_ptr(), too_many, 0, 0, 1.0, result.data_ptr(), 512, stream) == B.ERR_TOO_LARGE
    assert B.grad_norm_static(g16.data_ptr(), 4096, 0, 0, 1.0, result.data_ptr(), 1000, stream) == B.ERR_INVALID_ARG
    assert B.grad_norm_static(g16.data_ptr(), 4096, 0, 0, 1.0, 0, 0, stream) == B.ERR_INVALID_ARG
    assert B.grad_norm_static(g16.data_ptr(), -1, 0, 0, 1.0, result.data_ptr(), 0, stream) == B.ERR_INVALID_ARG
    assert B.grad_norm_static(g16.data_ptr() + 1, 16, 0, 0, 1.0, result.data_ptr(), 0, stream) == B.ERR_MISALIGNED
    assert B.grad_norm_static(g16.data_ptr(), 16, 0, 0, 1.0, result.data_ptr() + 4, 0, stream) == B.ERR_MISALIGNED
    assert B.grad_norm_static(0, 16, 0, 0, 1.0, result.data_ptr(), 0, stream) == B.ERR_INVALID_ARG
    torch.cuda.synchronize()


def test_static_norm_recorded_into_a_graph(B, torch_gpu):
    """What the entry point is for: recorded into a HIP graph (after one eager call on the device has looked up the
    scratch array's address) and replayed with new gradients; every replay equals the plan's norm of those gradients."""
    torch = torch_gpu
    n16, n32 = 200_003, 5_001
    g16 = torch.empty(n16, dtype=torch.float16, device="cuda:0")
    g32 = torch.empty(n32, dtype=torch.float32, device="cuda:0")
    result = torch.zeros(2, dtype=torch.float64, device="cuda:0")
    B.fill_f16(g16.data_ptr(), n16, 1, 0.0, 1e-3)
    B.fill_f32(g32.data_ptr(), n32, 2, 0.0, 1e-3)
    assert B.grad_norm_static(g16.data_ptr(), n16, g32.data_ptr(), n32, 0.25, result.data_ptr()) == B.OK
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            assert B.grad_norm_static(g16.data_ptr(), n16, g32.data_ptr(), n32, 0.25, result.data_ptr(), 0, s) == B.OK
    torch.cuda.synchronize()
    for k in range(4):
        B.fill_f16(g16.data_ptr(), n16, 10 + k, 0.0, 1e-3 * (k + 1))          # eager work between the replays
        B.fill_f32(g32.data_ptr(), n32, 20 + k, 0.0, 1e-3 * (k + 1))
        result.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = read_device(result.data_ptr(), 16).copy()
        want, _ = plan_result(B, g16, n16, g32, n32, 0, 0.25, 0)
        assert np.array_equal(got, want), k
