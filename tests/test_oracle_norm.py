"""Pins the oracle's gradient norm, clip rule, scale pass, reduction-order mirror and the seeded
generator.  The reference has no test of clip_grad_norm_ (include/training/trainer.h:323-352),
so these rest on numpy float64, known vectors and the rule's own definition."""
import numpy as np


def test_sum_sq_against_numpy_float64(O):
    g = O.fill_f16(1_000_003, 5, 0.0, 5e-3)
    x = g.view(np.float16).astype(np.float64)
    assert abs(O.sum_sq_half(g) - float(np.dot(x, x))) <= 1e-12 * float(np.dot(x, x))
    f = O.fill_f32(70_001, 6, 0.0, 2.0)
    y = f.astype(np.float64)
    assert abs(O.sum_sq_float(f) - float(np.dot(y, y))) <= 1e-12 * float(np.dot(y, y))


def test_known_vectors(O):
    ones = np.full(1 << 20, 0x3C00, np.uint16)                    # 1.0 in FP16
    assert O.sum_sq_half(ones) == float(1 << 20)
    norm, scale = O.clip_grad_norm(ones.copy(), None, 2048.0)
    assert norm == 1024.0 and scale == 1.0
    three_four = np.array([3.0, 4.0], np.float32)
    assert O.clip_grad_norm(None, three_four.copy(), 10.0)[0] == 5.0
    assert O.sum_sq_half(np.zeros(0, np.uint16)) == 0.0


def test_clip_rule(O):
    # strict '>' (trainer.h:343): a norm equal to max_norm is not scaled
    s, n = O.clip_scale(np.float32(25.0), 5.0)
    assert n == 5.0 and s == 1.0
    # scale = max / (norm + 1e-6f), all in FP32 (trainer.h:344)
    s, n = O.clip_scale(np.float32(26.0), 5.0)
    want_n = np.sqrt(np.float32(26.0))
    assert n == float(want_n) and s == float(np.float32(5.0) / (want_n + np.float32(1e-6)))
    # a NaN norm compares false: no scaling
    s, n = O.clip_scale(np.float32(np.nan), 1.0)
    assert np.isnan(n) and s == 1.0
    s, n = O.clip_scale(np.float32(np.inf), 1.0)
    assert np.isinf(n) and s == 0.0


def test_clip_leaves_small_gradients_alone_and_scales_large_ones(O):
    g16 = O.fill_f16(300_000, 7, 0.0, 1e-3)
    g32 = O.fill_f32(5_000, 8, 0.0, 1e-3)
    a16, a32 = g16.copy(), g32.copy()
    norm, scale = O.clip_grad_norm(a16, a32, 1.0)
    assert norm < 1.0 and scale == 1.0 and np.array_equal(a16, g16) and np.array_equal(a32, g32)
    norm, scale = O.clip_grad_norm(a16, a32, 0.1)
    truth = np.sqrt(np.sum(g16.view(np.float16).astype(np.float64) ** 2) + np.sum(g32.astype(np.float64) ** 2))
    assert abs(norm - truth) <= 1e-6 * truth and norm > 0.1
    # the scale pass re-rounds FP16 gradients (trainer.h:136-139); numpy's float16 does the same
    want16 = (g16.view(np.float16).astype(np.float32) * np.float32(scale)).astype(np.float16).view(np.uint16)
    assert np.array_equal(a16, want16)
    assert np.array_equal(a32, g32 * np.float32(scale))
    post, _ = O.clip_grad_norm(a16.copy(), a32.copy(), 1e9)
    assert abs(post - 0.1) < 2e-3 * 0.1


def test_fused_clip_equals_scale_pass_then_update(O):
    n = 65_537
    p, g = O.fill_f16(n, 9, 0.0, 0.02), O.fill_f16(n, 10, 0.0, 5e-3)
    w32, g32 = O.fill_f32(777, 11, 1.0, 0.01), O.fill_f32(777, 12, 0.0, 5e-3)
    args = (1e-3, 0.9, 0.999, 1e-8, 0.01, O.bias_correction(0.9, 1), O.bias_correction(0.999, 1))
    ga, g32a = g.copy(), g32.copy()
    norm, scale = O.clip_grad_norm(ga, g32a, 0.5)
    assert norm > 0.5
    pa, ma, va = p.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    O.adamw_fp16(None, pa, ga, ma, va, *args)
    wa, m32a, v32a = w32.copy(), np.zeros(777, np.float32), np.zeros(777, np.float32)
    O.adamw_fp32(wa, g32a, m32a, v32a, *args)
    pb, mb, vb = p.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    O.adamw_fp16(None, pb, g, mb, vb, *args, clip_scale=scale)
    wb, m32b, v32b = w32.copy(), np.zeros(777, np.float32), np.zeros(777, np.float32)
    O.adamw_fp32(wb, g32, m32b, v32b, *args, clip_scale=scale)
    assert np.array_equal(pa, pb) and np.array_equal(ma, mb) and np.array_equal(va, vb)
    assert np.array_equal(wa, wb) and np.array_equal(m32a, m32b) and np.array_equal(v32a, v32b)


def test_mirror_order_sum(O):
    """The device-order FP32 tree stays within 1e-6 of the FP64 truth, is permutation-invariant to
    that accuracy, scale-equivariant, and its partial count is ceil(n / chunk) per tensor."""
    g = O.fill_f16(3 * 8192 + 4321, 13, 0.0, 5e-3)
    f = O.fill_f32(2049, 14, 0.0, 1e-2)
    truth = O.sum_sq_half(g) + O.sum_sq_float(f)
    s, parts = O.sumsq_mirror([g, f], 8192)
    assert parts.size == 4 + 1 and abs(s - truth) <= 1e-6 * truth
    rng = np.random.default_rng(0)
    s2, _ = O.sumsq_mirror([np.ascontiguousarray(g[rng.permutation(g.size)]), f], 8192)
    assert abs(s2 - s) <= 1e-6 * s
    g4 = O.f2h(O.h2f(g) * np.float32(4.0))                          # exact scaling by a power of two
    s4, _ = O.sumsq_mirror([g4], 8192)
    s1, _ = O.sumsq_mirror([g], 8192)
    assert s4 == 16.0 * s1
    ones = np.full(1 << 20, 0x3C00, np.uint16)
    assert O.sumsq_mirror([ones], 2048)[0] == float(1 << 20)
    assert O.sumsq_mirror([ones[:5]], 2048)[0] == 5.0


def test_mirror_order_with_group_partials(O):
    """512-element chunks: 16 consecutive chunk partials are added, in order, into one group partial before the
    fixed-order sum.  Same pins as for the plain order (FP64 truth, known vectors, power-of-two scaling), plus the
    grouping itself against a plain Python loop."""
    rng = np.random.default_rng(1)
    sizes = [128, 1024, 513, 5000, 40000, 7, 65536, 129]
    grads = [O.fill_f16(n, 20 + i, 0.0, 1e-3) for i, n in enumerate(sizes)] + [O.fill_f32(3000, 99, 0.0, 1e-2)]
    truth = sum(O.sum_sq_half(g) if g.dtype == np.uint16 else O.sum_sq_float(g) for g in grads)
    s, parts = O.sumsq_mirror(grads, 512)
    assert parts.size == sum((g.size + 511) // 512 for g in grads)
    assert abs(s - truth) <= 1e-6 * truth
    groups = O.sumsq_mirror_groups(parts)
    assert groups.size == (parts.size + 15) // 16
    for k in range(groups.size):
        total = 0.0
        for x in parts[16 * k: 16 * k + 16]:
            total += float(x)                                       # Python floats are IEEE doubles
        assert groups[k] == total
    assert s == O.sumsq_mirror_final(groups) == O.sumsq_mirror_total(parts, 512)
    assert O.sumsq_mirror_total(parts, 2048) == O.sumsq_mirror_final(parts)       # no grouping for other chunk sizes
    g4 = [O.f2h(O.h2f(g) * np.float32(4.0)) if g.dtype == np.uint16 else g * np.float32(4.0) for g in grads]
    assert O.sumsq_mirror(g4, 512)[0] == 16.0 * s
    ones = np.full(100_000, 0x3C00, np.uint16)
    assert O.sumsq_mirror([ones], 512)[0] == 100_000.0
    assert O.sumsq_mirror([ones[:5]], 512)[0] == 5.0
    perm = [np.ascontiguousarray(g[rng.permutation(g.size)]) for g in grads]
    assert abs(O.sumsq_mirror(perm, 512)[0] - s) <= 1e-6 * s


def test_generator(O):
    a = O.fill_f16(100_000, 77, 0.0, 1e-3)
    assert np.array_equal(a, O.fill_f16(100_000, 77, 0.0, 1e-3))
    assert not np.array_equal(a, O.fill_f16(100_000, 78, 0.0, 1e-3))
    # `first` addresses the same stream: a window equals the slice
    assert np.array_equal(O.fill_f16(1000, 77, 0.0, 1e-3, first=4242), a[4242:5242])
    z = O.fill_f32(2_000_000, 79, 0.0, 1.0)
    assert abs(z.mean()) < 3e-3 and abs(z.std() - 1.0) < 3e-3 and np.abs(z).max() < 4.9
    assert abs(np.mean(z ** 3)) < 1e-2 and abs(np.mean(z ** 4) - 3.0) < 0.2
    y = O.fill_f32(100_000, 80, 2.0, 0.5, flags=O.FILL_ABS)
    assert y.min() >= 2.0
    # row mask: whole rows are zero, about the requested share of them
    rows, row_len = 4000, 64
    e = O.fill_f16(rows * row_len, 81, 0.0, 1e-2, row_len=row_len, zero_rows_below=int(0.9 * 2 ** 32))
    zero_rows = ~e.reshape(rows, row_len).any(axis=1)
    assert abs(zero_rows.mean() - 0.9) < 0.02
    assert (e.reshape(rows, row_len)[~zero_rows] != 0).mean() > 0.9


def test_tolerance_covers_the_reference_norm_in_any_atomic_order(O):
    """The reference adds up the gradient norm in FP32: every thread of a grid of at most 2048 x 256 strides over
    the buffer with one FP32 accumulator, a warp combines by xor shuffle (masks 16..1), and lane 0 of every warp
    adds its sum to one float with atomicAdd, in whatever order the warps arrive (include/training/trainer.h:103-117,
    327-337).  Its last bits therefore differ from run to run and cannot be reproduced.  What can be shown: that
    structure, replayed here in FP32 with the warps arriving in several random orders, stays within 1e-5 relative
    of the FP64 sum, and so does this path's fixed order, so the two always agree within the stated tolerance."""
    n = 1 << 24
    bits = O.fill_f16(n, 77, 0.0, 5e-3)
    x = O.h2f(bits)
    truth = float(np.dot(x.astype(np.float64), x.astype(np.float64)))
    threads = 2048 * 256
    sq = (x * x).reshape(n // threads, threads)
    acc = np.zeros(threads, np.float32)
    for row in sq:                                               # each thread: sum += v * v over its strided elements
        acc = acc + row
    warp = acc.reshape(-1, 32)
    lanes = np.arange(32)
    for mask in (16, 8, 4, 2, 1):                                # __shfl_xor_sync butterfly
        warp = warp + warp[:, lanes ^ mask]
    per_warp = warp[:, 0].copy()
    rng = np.random.default_rng(0)
    sums = []
    for _ in range(6):
        order = rng.permutation(per_warp.size)
        sums.append(float(np.cumsum(per_warp[order], dtype=np.float32)[-1]))      # atomicAdd, one at a time
    assert len(set(sums)) > 1                                    # the order does change the bits
    mine, _ = O.sumsq_mirror([bits], 8192)
    for s in sums + [mine]:
        assert abs(s - truth) <= 1e-5 * truth
        norm_ref, norm_mine = np.sqrt(np.float32(s)), np.sqrt(np.float32(mine))
        assert abs(float(norm_ref) - float(norm_mine)) <= 1e-5 * float(norm_mine)
    assert abs(mine - truth) <= 1e-6 * truth                     # the fixed order is the closer one
