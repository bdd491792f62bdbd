"""GPU parity of the multi-tensor plan (norm, clip, update) against the CPU oracle, through the
C ABI.  Sizes here are small enough for the oracle to replay every element."""
import os

import numpy as np
import pytest

from util import HYPER, bits, check_state, read_device

pytestmark = pytest.mark.gpu

MINI = dict(vocab=1000, hidden=64, inter=192, layers=2, q_heads=4, kv_heads=2, head_dim=16, tied=True)


def host_copy(store):
    """numpy copies of every tensor's p, g, m, v (and master)."""
    out = []
    for i in range(len(store.specs)):
        d = dict(p=bits(store.param(i)), g=bits(store.grad(i)), m=bits(store.state(i, "m")),
                 v=bits(store.state(i, "v")))
        if store.master is not None:
            d["master"] = bits(store.state(i, "master"))
        out.append(d)
    return out


def oracle_step(O, L, specs, hs, step, hyper, clip_scale=None, master=False):
    bc1, bc2 = O.bias_correction(hyper["beta1"], step), O.bias_correction(hyper["beta2"], step)
    for s, h in zip(specs, hs):
        wd = 0.0 if s.flags & L.NO_DECAY else hyper["wd"]
        if s.dtype == L.DTYPE_F16:
            O.adamw_fp16(h.get("master") if master else None, h["p"], h["g"], h["m"], h["v"], hyper["lr"],
                         hyper["beta1"], hyper["beta2"], hyper["eps"], wd, bc1, bc2, clip_scale=clip_scale)
        else:
            O.adamw_fp32(h["p"], h["g"], h["m"], h["v"], hyper["lr"], hyper["beta1"], hyper["beta2"],
                         hyper["eps"], wd, bc1, bc2, clip_scale=clip_scale)


def compare(store, hs, what=""):
    bad = 0
    for i, h in enumerate(hs):
        bad += check_state(bits(store.param(i)), bits(store.state(i, "m")), bits(store.state(i, "v")),
                           h["p"], h["m"], h["v"], "%s tensor %d" % (what, i))
        if "master" in h and store.specs[i].dtype == 0:
            assert np.array_equal(bits(store.state(i, "master")), h["master"])
    return bad


@pytest.mark.parametrize("norm_dtype,ref_groups,master", [(0, False, False), (1, True, False), (1, True, True)])
def test_model_shaped_list_five_steps(O, L, host, torch_gpu, norm_dtype, ref_groups, master):
    """A small Qwen3-shaped tensor list (all FP16, or the reference's layout with FP32 norm weights,
    no decay on embedding and norms, FP32 master copy), five steps with fresh gradients."""
    torch = torch_gpu
    specs = L.qwen3_tensor_list(MINI, norm_dtype=norm_dtype, reference_decay_groups=ref_groups)
    st = host.ParamStore(specs, master=master)
    st.fill("p", 1, 0.0, 0.02)
    if master:
        st.init_master()
    opt = host.AdamWOptimizer(st, lr=1e-3, weight_decay=0.01, chunk_elems=2048)
    hyper = dict(HYPER, lr=1e-3)
    torch.cuda.synchronize()
    hs = host_copy(st)
    bad = 0
    for step in range(1, 6):
        st.fill("g", 100 + step, 0.0, 1e-4, zero_row_frac=0.9, only=("embed_tokens",))
        torch.cuda.synchronize()
        for i, h in enumerate(hs):
            h["g"] = bits(st.grad(i))
        opt.step()
        assert opt.get_step() == step
        oracle_step(O, L, specs, hs, step, hyper, master=master)
        torch.cuda.synchronize()
        bad += compare(st, hs, "step %d" % step)
    assert bad == 0
    emb = [i for i, s in enumerate(specs) if s.name == "embed_tokens"][0]
    g = hs[emb]["g"].reshape(MINI["vocab"], MINI["hidden"])
    assert 0.8 < (~g.any(axis=1)).mean() < 0.97          # sparse token usage: most rows have zero gradient


def test_device_fill_equals_host_fill(O, L, host, torch_gpu):
    specs = [L.TensorSpec("e", 300 * 64, L.DTYPE_F16, 0, 64), L.TensorSpec("n", 1000, L.DTYPE_F32, 0, 0)]
    st = host.ParamStore(specs)
    st.fill("g", 9, 0.0, 1e-2, zero_row_frac=0.5, only=("e",))
    st.fill("m", 10, 1e-8, 1e-8, flags=1)
    torch_gpu.cuda.synchronize()
    thr = int(0.5 * 2 ** 32)
    assert np.array_equal(bits(st.grad(0)), O.fill_f16(300 * 64, L._hash64(9, 0), 0.0, 1e-2, row_len=64,
                                                       zero_rows_below=thr))
    assert np.array_equal(bits(st.grad(1)), O.fill_f32(1000, L._hash64(9, 1), 0.0, 1e-2))
    assert np.array_equal(bits(st.state(0, "m")), O.fill_f32(300 * 64, L._hash64(10, 0), 1e-8, 1e-8, flags=1))


def _norm_oracle(O, hs, chunk):
    truth = sum(O.sum_sq_half(h["g"]) if h["g"].dtype == np.uint16 else O.sum_sq_float(h["g"]) for h in hs)
    mirror, parts = O.sumsq_mirror([h["g"] for h in hs], chunk)
    return truth, mirror, parts


@pytest.mark.parametrize("chunk", [2048, 8192])
def test_grad_norm_and_clip(O, L, host, B, torch_gpu, chunk):
    """Norm within 1e-5 of the FP64 truth and bit-identical to the restated device order; the same
    bits on ten runs; fused clip == scale pass + plain step, bit for bit; scaled gradients equal the
    oracle's scale pass."""
    torch = torch_gpu
    specs = L.qwen3_tensor_list(MINI, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
    extra = torch.empty(777, dtype=torch.float32, device="cuda:0")           # a D_buf-like workspace tail
    B.fill_f32(extra.data_ptr(), 777, 5, 0.0, 0.3)
    stores, opts = [], []
    for _ in range(2):
        st = host.ParamStore(specs)
        st.fill("p", 1, 0.0, 0.02)
        st.fill("g", 2, 0.0, 5e-3)
        stores.append(st)
    ex2 = extra.clone()
    opts = [host.AdamWOptimizer(stores[0], lr=1e-3, chunk_elems=chunk, extra_grad_only=(extra,)),
            host.AdamWOptimizer(stores[1], lr=1e-3, chunk_elems=chunk, extra_grad_only=(ex2,))]
    torch.cuda.synchronize()
    hs = host_copy(stores[0])
    hs_all = hs + [dict(g=bits(extra))]
    truth, mirror, parts = _norm_oracle(O, hs_all, chunk)
    max_norm = 1.0
    seen = set()
    for _ in range(10):
        opts[0].plan.grad_norm(max_norm)
        seen.add(opts[0].plan.norm_read())
    assert len(seen) == 1, "norm differs between runs"
    norm, scale, sum_sq = seen.pop()
    assert abs(sum_sq - truth) <= 1e-5 * truth
    assert sum_sq == mirror, "device reduction order differs from its restatement"
    assert parts.size == opts[0].plan.num_chunks
    o_scale, o_norm = O.clip_scale(np.float32(truth), max_norm)
    assert abs(norm - o_norm) <= 1e-5 * o_norm and norm > max_norm
    assert scale == O.clip_scale(np.float32(sum_sq), max_norm)[0]
    # unfused: clip_grad_norm_ scales in place, then a plain step
    got_norm = opts[0].clip_grad_norm_(max_norm)
    assert got_norm == norm
    opts[0].step()
    # fused: gradients untouched, scale applied inside the update
    assert host.training_step(opts[1], max_norm, fused_clip=True) == norm
    torch.cuda.synchronize()
    for i in range(len(specs)):
        assert np.array_equal(bits(stores[1].grad(i)), hs[i]["g"]), "fused clip must not write gradients"
    assert np.array_equal(bits(ex2), hs_all[-1]["g"])
    # oracle: scale pass (both dtypes, workspace tail included), then the update
    for h in hs_all:
        if h["g"].dtype == np.uint16:
            O.scale_half(h["g"], scale)
        else:
            O.scale_float(h["g"], scale)
    for i in range(len(specs)):
        assert np.array_equal(bits(stores[0].grad(i)), hs[i]["g"]), "scaled gradients, tensor %d" % i
    assert np.array_equal(bits(extra), hs_all[-1]["g"])
    oracle_step(O, L, specs, hs, 1, dict(HYPER, lr=1e-3))
    assert compare(stores[0], hs, "unfused") == 0
    assert compare(stores[1], hs, "fused") == 0


@pytest.mark.parametrize("chunk", [512, 1024, 2048, 4096, 8192, 65536])
def test_norm_partials_on_wide_range_gradients(O, L, host, B, torch_gpu, chunk):
    """Gradients that are uniformly random finite FP16 bit patterns (magnitudes from 6e-8 to 65504, so FP32
    accumulators round at every addition) and FP32 gradients spread over forty binades: every per-chunk partial
    and the total equal the restated reduction order bit for bit, for each width of the norm workgroup."""
    torch = torch_gpu
    rng = np.random.default_rng(chunk)
    n16, n32 = 300_007, 70_001
    h = rng.integers(0, 1 << 16, n16, dtype=np.uint32).astype(np.uint16)
    h[(h & 0x7C00) == 0x7C00] &= 0x83FF                      # infinities and NaNs become subnormals
    f = (rng.standard_normal(n32) * np.exp2(rng.integers(-20, 20, n32))).astype(np.float32)
    g16 = torch.from_numpy(h.view(np.int16)).to("cuda:0").view(torch.float16)
    g32 = torch.from_numpy(f).to("cuda:0")
    descs = [B.TensorDesc(None, g16.data_ptr(), None, None, None, n16, B.DTYPE_F16, B.TENSOR_GRAD_ONLY),
             B.TensorDesc(None, g32.data_ptr(), None, None, None, n32, B.DTYPE_F32, B.TENSOR_GRAD_ONLY)]
    plan = B.Plan(descs, chunk)
    plan.grad_norm(1.0)
    norm, scale, sum_sq = plan.norm_read()
    mirror, parts = O.sumsq_mirror([h, f], chunk)
    assert parts.size == plan.num_chunks
    dev_parts = read_device(plan.partials_ptr, 8 * plan.num_chunks).view(np.float64)
    assert np.array_equal(dev_parts.view(np.uint64), parts.view(np.uint64)), "partials differ"
    assert sum_sq == mirror
    truth = float((O.h2f(h).astype(np.float64) ** 2).sum() + (f.astype(np.float64) ** 2).sum())
    assert abs(sum_sq - truth) <= 1e-5 * truth


def test_norm_below_threshold_touches_nothing(O, L, host, torch_gpu):
    torch = torch_gpu
    specs = [L.TensorSpec("a", 50_000, L.DTYPE_F16, 0, 0), L.TensorSpec("b", 333, L.DTYPE_F32, 0, 0)]
    st = host.ParamStore(specs)
    st.fill("g", 3, 0.0, 1e-4)
    opt = host.AdamWOptimizer(st)
    torch.cuda.synchronize()
    before = [bits(st.grad(i)) for i in range(2)]
    norm = opt.clip_grad_norm_(1.0)
    opt.plan.scale_grads()                       # even when called anyway: scale is exactly 1
    torch.cuda.synchronize()
    _, scale, _ = opt.plan.norm_read()
    assert 0 < norm < 1.0 and scale == 1.0
    assert all(np.array_equal(bits(st.grad(i)), before[i]) for i in range(2))


def test_non_finite_gradient(O, L, host, torch_gpu):
    """A NaN gradient gives a NaN norm; the comparison is false, so nothing is scaled
    (include/training/trainer.h:343) and the update propagates the NaN to that element only."""
    torch = torch_gpu
    specs = [L.TensorSpec("a", 5000, L.DTYPE_F16, 0, 0)]
    st = host.ParamStore(specs)
    st.fill("p", 1, 0.0, 0.02)
    st.fill("g", 2, 0.0, 1e-2)
    st.grad(0)[1234] = float("nan")
    opt = host.AdamWOptimizer(st, lr=1e-3)
    norm = host.training_step(opt, 1.0, fused_clip=True)
    torch.cuda.synchronize()
    _, scale, _ = opt.plan.norm_read()
    assert np.isnan(norm) and scale == 1.0
    p = st.param(0).float().cpu().numpy()
    assert np.isnan(p[1234]) and np.isfinite(np.delete(p, 1234)).all()


@pytest.mark.parametrize("fused", [False, True])
def test_infinite_gradient(O, L, host, torch_gpu, fused):
    """An infinite gradient gives an infinite norm and the scale max/(inf + 1e-6f) = 0
    (include/training/trainer.h:343-344): every finite gradient becomes a (signed) zero, the infinite one
    0 * inf = NaN, with the scale pass and fused alike; the oracle's two-step restatement agrees bit for bit
    on every finite result."""
    torch = torch_gpu
    n = 5000
    specs = [L.TensorSpec("a", n, L.DTYPE_F16, 0, 0)]
    st = host.ParamStore(specs)
    st.fill("p", 1, 0.0, 0.02)
    st.fill("g", 2, 0.0, 1e-2)
    st.grad(0)[777] = float("inf")
    torch.cuda.synchronize()
    p_h, g_h = bits(st.param(0)), bits(st.grad(0))
    m_h, v_h = np.zeros(n, np.float32), np.zeros(n, np.float32)
    opt = host.AdamWOptimizer(st, lr=1e-3)
    norm = host.training_step(opt, 1.0, fused_clip=fused)
    torch.cuda.synchronize()
    _, scale, _ = opt.plan.norm_read()
    assert np.isinf(norm) and scale == 0.0
    assert O.clip_scale(float("inf"), 1.0) == (0.0, float("inf"))
    O.scale_half(g_h, 0.0)
    O.adamw_fp16(None, p_h, g_h, m_h, v_h, 1e-3, 0.9, 0.999, 1e-8, 0.01, host.bias_correction(0.9, 1),
                 host.bias_correction(0.999, 1))
    got_p, got_m, got_v = bits(st.param(0)), bits(st.state(0, "m")), bits(st.state(0, "v"))
    keep = np.arange(n) != 777
    assert np.array_equal(got_p[keep], p_h[keep])
    assert np.array_equal(got_m[keep].view(np.uint32), m_h[keep].view(np.uint32))
    assert np.array_equal(got_v[keep].view(np.uint32), v_h[keep].view(np.uint32))
    assert np.isnan(got_m[777]) and np.isnan(m_h[777]) and (got_p[777] & 0x7FFF) > 0x7C00
    if not fused:
        g_after = bits(st.grad(0))
        assert np.array_equal(g_after[keep], g_h[keep]) and (g_after[777] & 0x7FFF) > 0x7C00


def test_ragged_list_equals_flat_tensor(O, L, host, B, torch_gpu):
    """4,096 tensors of 128..65,536 elements in one launch against one flat tensor with the same
    values: identical bits, and both equal to the oracle."""
    torch = torch_gpu
    specs = L.ragged_tensor_list()
    total = L.total_elements(specs)
    st = host.ParamStore(specs)
    st.fill("p", 1, 1.0, 0.01)
    st.fill("g", 2, 0.0, 1e-3)
    torch.cuda.synchronize()
    hs = host_copy(st)
    flat_p = torch.cat([st.param(i) for i in range(len(specs))]).contiguous()
    flat_g = torch.cat([st.grad(i) for i in range(len(specs))]).contiguous()
    flat_m = torch.zeros(total, dtype=torch.float32, device="cuda:0")
    flat_v = torch.zeros(total, dtype=torch.float32, device="cuda:0")
    opt = host.AdamWOptimizer(st, lr=1e-5)
    assert opt.plan.chunk_elems == 512                       # small-tensor lists get small chunks
    opt.step()
    bc1, bc2 = host.bias_correction(0.9, 1), host.bias_correction(0.999, 1)
    assert B.adamw_fp16(None, flat_p.data_ptr(), flat_g.data_ptr(), flat_m.data_ptr(), flat_v.data_ptr(), total,
                        1e-5, 0.9, 0.999, 1e-8, 0.01, bc1, bc2) == B.OK
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([st.param(i) for i in range(len(specs))]), flat_p)
    assert torch.equal(torch.cat([st.state(i, "m") for i in range(len(specs))]), flat_m)
    assert torch.equal(torch.cat([st.state(i, "v") for i in range(len(specs))]), flat_v)
    oracle_step(O, L, specs, hs, 1, dict(HYPER))
    assert compare(st, hs) == 0
    # padding between tensors is never written
    used = torch.zeros(st.m.numel(), dtype=torch.bool, device="cuda:0")
    for i, s in enumerate(specs):
        used[st.off[i]: st.off[i] + s.n] = True
    assert not st.m[~used].any().item() and not st.p16[~used[: st.p16.numel()]].any().item()


@pytest.mark.parametrize("master,zero_grads", [(False, False), (True, False), (False, True), (True, True)])
def test_every_tile_shape_and_chunk_size_gives_the_same_bits(L, host, B, torch_gpu, master, zero_grads):
    """Every compiled form of the update kernel (tile shapes, XCD swizzle, store policy, the two forms that
    issue their loads and stores at once or two at a time, and the 128-bit-access forms: one wavefront per tile,
    a persistent grid striding over the tiles, one workgroup walking a chunk, lane pairs sharing 128-bit accesses)
    gives the same bits, with and
    without a master copy and gradient clearing (which select between the first two forms by default)."""
    torch = torch_gpu
    specs = [L.TensorSpec("a", 70_001, L.DTYPE_F16, 0, 0), L.TensorSpec("b", 2049, L.DTYPE_F32, 0, 0),
             L.TensorSpec("c", 131, L.DTYPE_F16, L.NO_DECAY, 0)]
    results = []
    try:
        for variant, chunk in [(0, 8192), (1, 8192), (2, 2048), (3, 512), (4, 512), (5, 65536), (6, 1024),
                               (7, 2048), (8, 8192), (9, 4096), (10, 512), (10, 8192), (11, 512), (11, 2048),
                               (11, 65536), (12, 512), (12, 8192), (13, 2048), (14, 8192), (15, 512), (15, 8192),
                               (16, 512), (16, 1024), (16, 8192), (17, 512), (17, 2048), (17, 8192)]:
            B.set_tuning("update_variant", variant)
            st = host.ParamStore(specs, master=master)
            st.fill("p", 1, 0.0, 0.02)
            st.fill("g", 2, 0.0, 5e-3)
            if master:
                st.init_master()
            opt = host.AdamWOptimizer(st, lr=1e-3, chunk_elems=chunk)
            host.training_step(opt, 0.05, fused_clip=True, zero_grads=zero_grads)
            if zero_grads:
                assert not st.g16.any().item() and not st.g32.any().item()
                st.fill("g", 3, 0.0, 5e-3)
            host.training_step(opt, 0.0)
            torch.cuda.synchronize()
            results.append([t.clone() for t in (st.p16, st.p32, st.m, st.v)] + ([st.master.clone()] if master else []))
    finally:
        B.set_tuning("update_variant", 0)
    for r in results[1:]:
        assert all(torch.equal(a, b) for a, b in zip(results[0], r))


def test_cache_aware_orders_give_the_same_bits(L, host, B, torch_gpu):
    """The two orders meant to let the update find the gradients that the norm read last still in the last-level
    cache (the norm walking its chunks backwards with ordinary loads on the stretch it reads last; the fused-clip
    update walking its tiles backwards) change neither the norm's result nor any bit of the state: every chunk's
    partial keeps its slot, every tile its arithmetic."""
    torch = torch_gpu
    specs = [L.TensorSpec("a", 300_001, L.DTYPE_F16, 0, 0), L.TensorSpec("b", 2049, L.DTYPE_F32, 0, 0),
             L.TensorSpec("c", 131, L.DTYPE_F16, L.NO_DECAY, 0), L.TensorSpec("d", 9000, L.DTYPE_F16, 0, 0)]
    results = {}
    try:
        for chunk in (8192, 1024):
            for keep_mb, reverse in [(0, 0), (1, 0), (0, 1), (1, 1), (4096, 1)]:
                B.set_tuning("norm_keep_mb", keep_mb)
                B.set_tuning("update_reverse", reverse)
                st = host.ParamStore(specs)
                st.fill("p", 1, 0.0, 0.02)
                st.fill("g", 2, 0.0, 5e-3)
                opt = host.AdamWOptimizer(st, lr=1e-3, chunk_elems=chunk)
                norm = host.training_step(opt, 0.05, fused_clip=True)
                st.fill("g", 3, 0.0, 5e-3)
                norm2 = host.training_step(opt, 0.05, fused_clip=True, zero_grads=True)
                torch.cuda.synchronize()
                results[(chunk, keep_mb, reverse)] = (np.float32(norm), np.float32(norm2),
                                                      [t.clone() for t in (st.p16, st.p32, st.m, st.v)])
    finally:
        B.set_tuning("norm_keep_mb", 0)
        B.set_tuning("update_reverse", 0)
    for (chunk, keep_mb, reverse), (norm, norm2, state) in results.items():
        base = results[(chunk, 0, 0)]                    # the order of the sum, and so its bits, belong to the chunk size
        assert norm == base[0] and norm2 == base[1], (chunk, keep_mb, reverse)
        assert all(torch.equal(a, b) for a, b in zip(base[2], state)), (chunk, keep_mb, reverse)


def test_unaligned_tensors_in_a_plan(O, L, host, B, torch_gpu):
    """Tensors that start at odd element offsets take the element-by-element path."""
    torch = torch_gpu
    n = 10_001
    pool_p = torch.empty(n + 8, dtype=torch.float16, device="cuda:0")
    pool_g = torch.empty(n + 8, dtype=torch.float16, device="cuda:0")
    pool_m = torch.zeros(n + 8, dtype=torch.float32, device="cuda:0")
    pool_v = torch.zeros(n + 8, dtype=torch.float32, device="cuda:0")
    B.fill_f16(pool_p.data_ptr(), n + 8, 1, 0.0, 0.02)
    B.fill_f16(pool_g.data_ptr(), n + 8, 2, 0.0, 5e-3)
    torch.cuda.synchronize()
    hp, hg = bits(pool_p), bits(pool_g)
    hm, hv = np.zeros(n + 8, np.float32), np.zeros(n + 8, np.float32)
    off = 3
    d = B.TensorDesc(pool_p.data_ptr() + 2 * off, pool_g.data_ptr() + 2 * off, pool_m.data_ptr() + 4 * off,
                     pool_v.data_ptr() + 4 * off, None, n, B.DTYPE_F16, 0)
    plan = B.Plan([d], 2048)
    plan.grad_norm(0.1)
    norm, scale, sum_sq = plan.norm_read()
    assert sum_sq == O.sumsq_mirror([hg[off: off + n]], 2048)[0]
    sp = B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.01, host.bias_correction(0.9, 1), host.bias_correction(0.999, 1))
    plan.adamw(sp, B.CLIP_FUSED)
    torch.cuda.synchronize()
    sl = slice(off, off + n)
    O.adamw_fp16(None, hp[sl], hg[sl], hm[sl], hv[sl], 1e-3, 0.9, 0.999, 1e-8, 0.01, sp.bias_correction1,
                 sp.bias_correction2, clip_scale=scale)
    assert np.array_equal(bits(pool_p), hp) and np.array_equal(bits(pool_m), hm) and np.array_equal(bits(pool_v), hv)
    plan.destroy()


def test_zero_grads_in_the_update_and_frozen_embedding(O, L, host, B, torch_gpu):
    """The reference's step is: clear all gradients (qwen3.cu:1109-1112), accumulate, clear the frozen
    embedding's gradients (trainer.h:269-277), clip, update.  Here the frozen tensor is flagged in the
    plan and the update clears every gradient buffer after reading it.  Weights, moments and the norm
    must come out as in the reference's order of operations, and all gradient buffers must be zero."""
    torch = torch_gpu
    ref_specs = L.qwen3_tensor_list(MINI, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
    frz_specs = L.qwen3_tensor_list(MINI, norm_dtype=L.DTYPE_F32, reference_decay_groups=True, freeze_embed=True)
    emb = [i for i, s in enumerate(ref_specs) if s.name == "embed_tokens"][0]
    assert frz_specs[emb].flags & L.FROZEN
    st_a, st_b = host.ParamStore(ref_specs), host.ParamStore(frz_specs)
    tails = [torch.empty(555, dtype=torch.float32, device="cuda:0") for _ in range(2)]
    opt_a = host.AdamWOptimizer(st_a, lr=1e-3, chunk_elems=2048, extra_grad_only=(tails[0],))
    opt_b = host.AdamWOptimizer(st_b, lr=1e-3, chunk_elems=2048, extra_grad_only=(tails[1],))
    for st in (st_a, st_b):
        st.fill("p", 1, 0.0, 0.02)
    torch.cuda.synchronize()
    hs = host_copy(st_a)
    for step in range(1, 4):
        st_a.zero_grads()                                        # qwen3_gradients_zero, then "backward":
        assert not st_a.g16.any().item() and not st_a.g32.any().item()
        for st, tail in ((st_a, tails[0]), (st_b, tails[1])):
            st.fill("g", 50 + step, 0.0, 5e-3)
            B.fill_f32(tail.data_ptr(), 555, 60 + step, 0.0, 0.1)
        B.clear(st_a.grad(emb).data_ptr(), ref_specs[emb].n * 2)  # the reference's freeze_embed memset
        torch.cuda.synchronize()
        for i, h in enumerate(hs):
            h["g"] = bits(st_a.grad(i))
        tail_h = bits(tails[0])
        na = host.training_step(opt_a, 0.5, fused_clip=True)
        nb = host.training_step(opt_b, 0.5, fused_clip=True, zero_grads=True)
        torch.cuda.synchronize()
        assert na == nb and na > 0.5
        _, scale, _ = opt_b.plan.norm_read()
        oracle_step(O, L, ref_specs, hs, step, dict(HYPER, lr=1e-3), clip_scale=scale)
        assert compare(st_a, hs, "reference order, step %d" % step) == 0
        assert compare(st_b, hs, "frozen + zeroing, step %d" % step) == 0
        assert not st_b.g16.any().item() and not st_b.g32.any().item() and not tails[1].any().item()
        assert np.array_equal(bits(tails[0]), tail_h)            # without the flag nothing is cleared
    assert not st_b.state(emb, "m").any().item() and not st_b.state(emb, "v").any().item()


def test_device_resident_step_params_and_graph_replay(O, L, host, B, torch_gpu):
    """norm + fused-clip update recorded once as a HIP graph and replayed for several steps; between
    replays the host rewrites the 28 bytes of hyper-parameters on the device and new gradients arrive.
    Every replay is checked against the oracle, with eager work and synchronisations in between."""
    torch = torch_gpu
    specs = L.qwen3_tensor_list(MINI, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
    st = host.ParamStore(specs)
    st.fill("p", 1, 0.0, 0.02)
    st.fill("g", 2, 0.0, 5e-3)
    opt = host.AdamWOptimizer(st, lr=1e-3, chunk_elems=2048)
    torch.cuda.synchronize()
    hs = host_copy(st)
    dev_params = torch.zeros(7, dtype=torch.float32, device="cuda:0")
    pinned = torch.zeros(7, dtype=torch.float32).pin_memory()

    def set_params(step, lr):
        sp = B.StepParams(lr, 0.9, 0.999, 1e-8, 0.01, host.bias_correction(0.9, step),
                          host.bias_correction(0.999, step))
        pinned.copy_(torch.frombuffer(bytearray(bytes(sp)), dtype=torch.float32))
        dev_params.copy_(pinned, non_blocking=True)

    side = torch.cuda.Stream()
    set_params(1, 1e-3)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            opt.plan.grad_norm(0.5, s)
            opt.plan.adamw_dev(dev_params.data_ptr(), B.CLIP_FUSED, s)
    torch.cuda.synchronize()
    for step in range(1, 6):
        lr = 1e-3 / step
        if step > 1:
            st.fill("g", 2 + step, 0.0, 5e-3 * step)             # eager work between replays
            torch.cuda.synchronize()
            for i, h in enumerate(hs):
                h["g"] = bits(st.grad(i))
        set_params(step, lr)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        norm, scale, sum_sq = opt.plan.norm_read()
        truth = sum(O.sum_sq_half(h["g"]) if h["g"].dtype == np.uint16 else O.sum_sq_float(h["g"]) for h in hs)
        assert abs(sum_sq - truth) <= 1e-5 * truth and norm > 0.5
        assert sum_sq == O.sumsq_mirror([h["g"] for h in hs], 2048)[0]
        oracle_step(O, L, specs, hs, step, dict(HYPER, lr=lr), clip_scale=scale)
        assert compare(st, hs, "replay %d" % step) == 0


def test_scheduled_steps_replay_without_the_host(O, L, host, B, torch_gpu):
    """norm + fused-clip update + advance recorded once as a HIP graph; the hyper-parameters of six steps (a
    decaying learning rate, host-computed bias corrections) are uploaded once, and the graph is replayed five
    times with NO host write of hyper-parameters in between: only new gradients arrive (eager fills and
    synchronisations between the replays).  Every replay equals the oracle; the sixth, eager, scheduled step
    uses the sixth entry; the host mirror refuses a seventh; launched through the C ABI all the same, it reuses
    the last entry (the table is exhausted), the position saturates and the overrun is counted."""
    torch = torch_gpu
    specs = L.qwen3_tensor_list(MINI, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
    st = host.ParamStore(specs)
    st.fill("p", 1, 0.0, 0.02)
    st.fill("g", 2, 0.0, 5e-3)
    opt = host.AdamWOptimizer(st, lr=1e-3, chunk_elems=2048)
    torch.cuda.synchronize()
    hs = host_copy(st)
    lrs = [1e-3 / k for k in range(1, 7)]
    # a table with a zero bias correction or a non-finite rate is refused and changes nothing
    bad = [B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.01, 0.1, 0.0)]
    with pytest.raises(B.RlxError) as err:
        opt.plan.schedule_upload(bad)
    assert err.value.status == B.ERR_BAD_HYPER
    with pytest.raises(B.RlxError):
        opt.plan.adamw_scheduled()                               # no table yet
    opt.upload_schedule(lrs)
    assert opt.plan.schedule_position() == (0, 6)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            opt.plan.grad_norm(0.5, s)
            opt.plan.adamw_scheduled(B.CLIP_FUSED, s)
    torch.cuda.synchronize()
    assert opt.plan.schedule_position() == (0, 6)                # capturing ran nothing

    def check(step, lr):
        norm, scale, sum_sq = opt.plan.norm_read()
        assert sum_sq == O.sumsq_mirror([h["g"] for h in hs], 2048)[0] and norm > 0.5
        oracle_step(O, L, specs, hs, step, dict(HYPER, lr=lr), clip_scale=scale)
        assert compare(st, hs, "scheduled step %d" % step) == 0

    for step in range(1, 6):
        if step > 1:
            st.fill("g", 2 + step, 0.0, 5e-3 * step)             # new gradients: the only thing the host provides
            torch.cuda.synchronize()
            for i, h in enumerate(hs):
                h["g"] = bits(st.grad(i))
        graph.replay()
        torch.cuda.synchronize()
        check(step, lrs[step - 1])
        assert opt.plan.schedule_position() == (step, 6)
    # eager scheduled steps continue where the replays left off
    assert opt.get_step() == 0                                   # recording counted nothing
    opt.note_replayed_steps(5)
    assert opt.get_step() == 5 and opt.plan.schedule_overrun() == 0
    for step, lr in ((6, lrs[5]), (7, lrs[5])):
        opt.plan.grad_norm(0.5)
        if step == 6:
            opt.step_scheduled(fused_clip=True)
            torch.cuda.synchronize()
            check(6, lr)
            assert opt.plan.schedule_position() == (6, 6) and opt.get_step() == 6
            assert opt.plan.schedule_overrun() == 0
            with pytest.raises(RuntimeError):
                opt.step_scheduled(fused_clip=True)              # the table is used up: the mirror refuses
            assert opt.get_step() == 6
        else:
            opt.plan.adamw_scheduled(B.CLIP_FUSED)
            torch.cuda.synchronize()
            # exhausted: the last entry (step 6's bias corrections and rate) is used again
            norm, scale, _ = opt.plan.norm_read()
            bc1, bc2 = O.bias_correction(0.9, 6), O.bias_correction(0.999, 6)
            for s_, h in zip(specs, hs):
                wd = 0.0 if s_.flags & L.NO_DECAY else 0.01
                fn = O.adamw_fp16 if s_.dtype == L.DTYPE_F16 else O.adamw_fp32
                args = (None,) if s_.dtype == L.DTYPE_F16 else ()
                fn(*args, h["p"], h["g"], h["m"], h["v"], lr, 0.9, 0.999, 1e-8, wd, bc1, bc2, clip_scale=scale)
            assert compare(st, hs, "step beyond the table") == 0
            assert opt.plan.schedule_position() == (6, 6)
            assert opt.plan.schedule_overrun() == 1
    # a new upload starts again at its first entry
    opt.upload_schedule([2e-4])
    assert opt.plan.schedule_position() == (0, 1) and opt.plan.schedule_overrun() == 0


@pytest.mark.parametrize("norm_fused", [2, 0])
def test_one_recorded_step_replays_through_three_uploaded_windows(O, L, host, B, torch_gpu, norm_fused, request):
    """The reference sets a new learning rate from its scheduler before every step of the whole run
    (include/training/trainer.h:193-194, optimizer.h:120-122).  Here: norm + fused-clip scheduled update recorded
    ONCE as a HIP graph after the first upload, then replayed through window 1 (3 steps), a LONGER window 2
    (7 steps, the table is reallocated) and a shorter window 3 (2 steps), with nothing but the uploads and new
    gradients coming from the host.  Every one of the 12 steps equals the oracle's step with the scheduler's rate
    and the bias corrections of its step number; the position is right after every step and never passes the
    table's length; no step overruns its table."""
    torch = torch_gpu
    B.set_tuning("norm_fused", norm_fused)       # the norm's sum recorded as the tail of its launch, or as a second launch
    request.addfinalizer(lambda: B.set_tuning("norm_fused", 2))
    specs = L.qwen3_tensor_list(MINI, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
    st = host.ParamStore(specs)
    st.fill("p", 1, 0.0, 0.02)
    st.fill("g", 2, 0.0, 5e-3)
    opt = host.AdamWOptimizer(st, lr=1e-3, chunk_elems=2048)
    sched = host.LRScheduler()
    sched.init_cosine(1e-3, 1e-5, 2, 12)
    torch.cuda.synchronize()
    hs = host_copy(st)
    windows = [3, 7, 2]
    side = torch.cuda.Stream()
    graph = None
    step = 0
    for w, n in enumerate(windows):
        lrs = [sched.get_lr(step + k) for k in range(n)]        # the rate of global step step+k, as trainer.h:193
        assert opt.get_step() == step
        opt.upload_schedule(lrs)
        assert opt.plan.schedule_position() == (0, n)
        if graph is None:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    s = torch.cuda.current_stream().cuda_stream
                    opt.plan.grad_norm(0.5, s)
                    opt.step_scheduled(fused_clip=True, stream=s)
            torch.cuda.synchronize()
            assert opt.get_step() == 0 and opt.plan.schedule_position() == (0, n)      # recording ran nothing
        for k in range(n):
            step += 1
            st.fill("g", 100 + step, 0.0, 2e-3 * step)
            torch.cuda.synchronize()
            for i, h in enumerate(hs):
                h["g"] = bits(st.grad(i))
            graph.replay()
            torch.cuda.synchronize()
            norm, scale, sum_sq = opt.plan.norm_read()
            assert sum_sq == O.sumsq_mirror([h["g"] for h in hs], 2048)[0] and norm > 0.5
            oracle_step(O, L, specs, hs, step, dict(HYPER, lr=lrs[k]), clip_scale=scale)
            assert compare(st, hs, "window %d step %d" % (w, step)) == 0
            taken, total = opt.plan.schedule_position()
            assert (taken, total) == (k + 1, n) and taken <= total                     # bounds of the table
            assert opt.plan.schedule_overrun() == 0
        opt.note_replayed_steps(n)
    assert opt.get_step() == 12 and abs(opt.lr - sched.get_lr(11)) == 0.0


def test_packed_norm_pass_gives_the_same_partials(O, L, host, B, torch_gpu):
    """512-element chunks: the forms of the first pass that give a workgroup 32, 16, 8 or one chunk, and every
    load depth of the second pass, write the same per-chunk partials and the same result, equal to the
    restated order; FP32 tensors, sizes that are no multiple of 8, and a frozen tensor included."""
    torch = torch_gpu
    specs = L.ragged_tensor_list(count=300, seed=11)
    specs += [L.TensorSpec("f32.%d" % i, n, L.DTYPE_F32, 0, 0) for i, n in enumerate((1, 3, 4, 5, 8, 509, 512, 513, 1027))]
    specs += [L.TensorSpec("frozen", 700, L.DTYPE_F16, L.FROZEN, 0)]
    st = host.ParamStore(specs)
    st.fill("g", 7, 0.0, 3e-3)
    opt = host.AdamWOptimizer(st, lr=1e-3, chunk_elems=512)
    torch.cuda.synchronize()
    grads = [bits(st.grad(i)) for i in range(len(specs))]
    grads[-1] = np.zeros_like(grads[-1])                         # a frozen tensor's gradients count as zero
    want, parts = O.sumsq_mirror(grads, 512)
    got = {}
    try:
        for pack, batch in ((2, 16), (3, 8), (1, 32), (0, 40)):
            B.set_tuning("norm_pack", pack)
            B.set_tuning("final_batch", batch)
            opt.plan.grad_norm(1.0)
            _, _, sum_sq = opt.plan.norm_read()
            got[pack] = (sum_sq, read_device(opt.plan.partials_ptr, 8 * opt.plan.num_chunks).view(np.float64).copy())
    finally:
        B.set_tuning("norm_pack", 3)
        B.set_tuning("final_batch", 0)
    for pack in got:
        assert got[pack][0] == want, pack
        assert np.array_equal(got[pack][1], parts), pack


@pytest.mark.parametrize("chunk,sizes", [
    (512, [128, 1024, 513, 7, 65536, 129, 300_000]),             # 512-element chunks: group partials, 19 workgroups
    (512, [512 * 32 * 64]),                                      # exactly 64 workgroups: one full ticket group
    (512, [512 * 32 * 65 + 1]),                                  # 66 workgroups: a second, short ticket group
    (1024, [1024 * 63, 5, 1024 * 2 + 1]),                        # 128-lane workgroups, 67 of them
    (2048, [2048 * 200 + 3, 100]),                               # 256-lane workgroups
    (8192, [8192 * 4100 + 77, 9000]),                            # 4,103 workgroups: beyond the automatic limit
    (8192, [1]),                                                 # a single workgroup is its own last one
    (1024, [1024 * 8192]),                                       # 8,192 workgroups: the largest one-launch grid
    (1024, [1024 * 8192 + 1]),                                   # 8,193: one more, always a second launch
])
def test_norm_summed_by_the_last_workgroup_equals_the_second_launch(O, B, torch_gpu, chunk, sizes):
    """The fixed-order sum of the partials as the tail of the first launch (the workgroup that draws the last
    ticket adds them) against the same sum as a second launch: identical 16 result bytes, identical partials,
    both equal to the restated order; three calls back to back each way (the tickets must be back at zero after
    every call), also with the chunks spread over fewer workgroups, through a plan and through the entry point
    that allocates nothing."""
    torch = torch_gpu
    stream = torch.cuda.current_stream().cuda_stream
    grads = []
    for i, n in enumerate(sizes):
        if i % 3 == 2:
            g = torch.empty(n, dtype=torch.float32, device="cuda:0")
            B.fill_f32(g.data_ptr(), n, 50 + i, 0.0, 2e-3)
        else:
            g = torch.empty(n, dtype=torch.float16, device="cuda:0")
            B.fill_f16(g.data_ptr(), n, 50 + i, 0.0, 5e-3)
        grads.append(g)
    torch.cuda.synchronize()
    host_g = [bits(g) for g in grads]
    want, parts = O.sumsq_mirror(host_g, chunk)
    scale, norm = O.clip_scale(np.float32(want), 0.01)
    descs = [B.TensorDesc(None, g.data_ptr(), None, None, None, g.numel(),
                          B.DTYPE_F16 if g.dtype == torch.float16 else B.DTYPE_F32, B.TENSOR_GRAD_ONLY) for g in grads]
    plan = B.Plan(descs, chunk)
    assert plan.num_chunks == parts.size
    results = {}
    try:
        for fused, grid in ((0, 0), (1, 0), (2, 0), (1, 3), (1, 64), (0, 3)):
            B.set_tuning("norm_fused", fused)
            B.set_tuning("norm_grid", grid)
            for rep in range(3):
                # every call sees new values (all gradients doubled, which multiplies every partial and the sum
                # by exactly 4): a sum that picked up a partial of the call before would show
                plan.grad_norm(0.01, stream)
                res = read_device(plan.norm_ptr, 16).copy()
                dev_parts = read_device(plan.partials_ptr, 8 * plan.num_chunks).view(np.float64).copy()
                assert np.array_equal(dev_parts, parts * 4.0 ** rep), (fused, grid, rep)
                assert res.view(np.float64)[0] == want * 4.0 ** rep, (fused, grid, rep)
                if rep == 0:
                    results[(fused, grid)] = res
                    if chunk == 512:
                        groups = read_device(plan.partials_ptr + 8 * plan.num_chunks, 8 * ((plan.num_chunks + 15) // 16))
                        assert np.array_equal(groups.view(np.float64), O.sumsq_mirror_groups(parts)), (fused, grid)
                for g in grads:
                    g.mul_(2.0)
            for g in grads:
                g.mul_(0.125)
    finally:
        B.set_tuning("norm_fused", 2)
        B.set_tuning("norm_grid", 0)
    for key, res in results.items():
        assert res.view(np.float64)[0] == want, key
        assert res.view(np.float32)[2] == np.float32(norm) and res.view(np.float32)[3] == np.float32(scale), key
    plan.destroy()
    # the same through rlx_grad_norm_static (always the second launch, whatever the tuning says): one FP16 buffer,
    # then one FP32 buffer
    h = [g for g in grads if g.dtype == torch.float16][0]
    f = ([g for g in grads if g.dtype == torch.float32] or [None])[0]
    out = torch.zeros((6, 2), dtype=torch.float64, device="cuda:0")
    try:
        for k, fused in enumerate((0, 1, 0, 1, 1, 0)):
            B.set_tuning("norm_fused", fused)
            assert B.grad_norm_static(h.data_ptr(), h.numel(), f.data_ptr() if f is not None else 0,
                                      f.numel() if f is not None else 0, 0.01, out[k].data_ptr(), chunk, stream) == B.OK
    finally:
        B.set_tuning("norm_fused", 2)
    torch.cuda.synchronize()
    two = [bits(h)] + ([bits(f)] if f is not None else [])
    want2, _ = O.sumsq_mirror(two, chunk)
    for k in range(6):
        assert read_device(out[k].data_ptr(), 8).view(np.float64)[0] == want2, k


def test_last_workgroup_sum_sees_every_partial_of_its_own_launch(B, torch_gpu):
    """The one-launch norm relies on device-scope stores, a wait and relaxed tickets instead of a full fence: a
    partial that the last workgroup read too early, or out of a cache, would be the value of the launch before.
    300 launches on gradients that change every time (a new seed and a new scale, so every chunk's partial moves),
    each followed at once by a fused-clip update that reads the scale, and each compared with the second-launch
    form on the same gradients: all 16 result bytes identical every time."""
    torch = torch_gpu
    stream = torch.cuda.current_stream().cuda_stream
    n = 8192 * 200 + 123                                          # 201 workgroups: four ticket groups, the last short
    p = torch.zeros(n, dtype=torch.float16, device="cuda:0")
    g = torch.empty(n, dtype=torch.float16, device="cuda:0")
    m = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    v = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    plan = B.Plan([B.TensorDesc(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), None, n, B.DTYPE_F16, 0)], 8192)
    sp = B.StepParams(1e-4, 0.9, 0.999, 1e-8, 0.0, 0.1, 0.001)
    seen = set()
    try:
        for k in range(300):
            B.fill_f16(g.data_ptr(), n, 1000 + k, 0.0, 1e-3 * (1 + k % 7), stream=stream)
            B.set_tuning("norm_fused", 1)
            plan.grad_norm(0.5, stream)
            plan.adamw(sp, B.CLIP_FUSED, stream)                  # reads the scale the moment the norm has finished
            one = read_device(plan.norm_ptr, 16).copy()
            B.set_tuning("norm_fused", 0)
            plan.grad_norm(0.5, stream)
            two = read_device(plan.norm_ptr, 16).copy()
            assert np.array_equal(one, two), (k, one.view(np.float64)[0], two.view(np.float64)[0])
            seen.add(float(one.view(np.float64)[0]))
    finally:
        B.set_tuning("norm_fused", 2)
    assert len(seen) == 300                                       # the sums did change from launch to launch
    plan.destroy()


def test_norm_takes_the_wide_path_from_the_gradient_alignment_alone(O, L, host, B, torch_gpu):
    """Gradients on a 16-byte boundary whose moments (and weights) start 4 bytes past one: the norm and the scale
    pass, which touch only the gradients, must not be pushed onto their element-by-element paths by the other
    streams' alignment, and the update must still take its own narrower path; everything equals the oracle."""
    torch = torch_gpu
    n = 50_000
    p = torch.zeros(n + 8, dtype=torch.float16, device="cuda:0")
    g = torch.zeros(n + 8, dtype=torch.float16, device="cuda:0")
    m = torch.zeros(n + 8, dtype=torch.float32, device="cuda:0")
    v = torch.zeros(n + 8, dtype=torch.float32, device="cuda:0")
    B.fill_f16(p.data_ptr(), n + 8, 1, 0.0, 0.02)
    B.fill_f16(g.data_ptr(), n + 8, 2, 0.0, 5e-3)
    torch.cuda.synchronize()
    assert g.data_ptr() % 16 == 0 and m.data_ptr() % 16 == 0
    # gradient aligned; weights 2 bytes, moments 4 bytes past a 16-byte boundary
    d = B.TensorDesc(p.data_ptr() + 2, g.data_ptr(), m.data_ptr() + 4, v.data_ptr() + 4, None, n, B.DTYPE_F16, 0)
    plan = B.Plan([d], 2048)
    p_before = bits(p)
    hp, hg = p_before[1: n + 1].copy(), bits(g)[:n].copy()
    hm, hv = np.zeros(n, np.float32), np.zeros(n, np.float32)
    want, parts = O.sumsq_mirror([hg], 2048)
    plan.grad_norm(0.25)
    norm, scale, sum_sq = plan.norm_read()
    assert sum_sq == want and norm > 0.25
    assert np.array_equal(read_device(plan.partials_ptr, 8 * plan.num_chunks).view(np.float64), parts)
    sp = B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.01, O.bias_correction(0.9, 1), O.bias_correction(0.999, 1))
    plan.adamw(sp, B.CLIP_FUSED)
    O.adamw_fp16(None, hp, hg, hm, hv, 1e-3, 0.9, 0.999, 1e-8, 0.01, sp.bias_correction1, sp.bias_correction2,
                 clip_scale=scale)
    torch.cuda.synchronize()
    assert np.array_equal(bits(p)[1: n + 1], hp)
    assert np.array_equal(bits(m)[1: n + 1], hm) and np.array_equal(bits(v)[1: n + 1], hv)
    assert bits(p)[0] == p_before[0] and np.array_equal(bits(p)[n + 1:], p_before[n + 1:])  # neighbours untouched
    assert bits(m)[0] == 0.0 and bits(m)[n + 1] == 0.0 and bits(v)[0] == 0.0 and bits(v)[n + 1] == 0.0
    plan.scale_grads()
    O.scale_half(hg, scale)
    torch.cuda.synchronize()
    assert np.array_equal(bits(g)[:n], hg)
    plan.destroy()


@pytest.mark.parametrize("n,src_off,dst_off", [(1 << 20, 0, 0), (2048 * 5 + 777, 0, 0), (300_001, 1, 0), (300_001, 0, 1),
                                               (4097, 4, 4), (100, 0, 0), (2048, 2, 2)])
def test_fp16_to_fp32_every_form(O, B, torch_gpu, n, src_off, dst_off):
    """The master-copy initialisation dst[i] = (float)src[i] (optimizer.h:46-57) in its four compiled forms, for
    whole and ragged sizes and for starts that are not aligned for the wide accesses: identical to the oracle's
    conversion, and nothing written outside [dst, dst + n)."""
    torch = torch_gpu
    src = torch.empty(n + 16, dtype=torch.float16, device="cuda:0")
    B.fill_f16(src.data_ptr(), n + 16, 31, 0.0, 3.0)
    want = O.h2f(bits(src)[src_off: src_off + n])
    try:
        for variant in (0, 1, 2, 3):
            B.set_tuning("convert_variant", variant)
            dst = torch.full((n + 16,), -7.0, dtype=torch.float32, device="cuda:0")
            assert B.fp16_to_fp32(dst.data_ptr() + 4 * dst_off, src.data_ptr() + 2 * src_off, n) == B.OK
            torch.cuda.synchronize()
            out = dst.cpu().numpy()
            assert np.array_equal(out[dst_off: dst_off + n].view(np.uint32), want.view(np.uint32)), variant
            assert (out[:dst_off] == -7.0).all() and (out[dst_off + n:] == -7.0).all(), variant
    finally:
        B.set_tuning("convert_variant", 0)


def test_plan_launches_on_its_own_device_after_a_device_round_trip(B, torch_gpu):
    """The device check that guards every plan launch (RLX_ERR_WRONG_DEVICE when another device is current) lets
    the owning device through, also after the current device has been set again explicitly."""
    torch = torch_gpu
    n = 4096
    p = torch.zeros(n, dtype=torch.float16, device="cuda:0"); g = torch.ones_like(p)
    m = torch.zeros(n, dtype=torch.float32, device="cuda:0"); v = torch.zeros_like(m)
    plan = B.Plan([B.TensorDesc(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), None, n, B.DTYPE_F16, 0)])
    lib = B.load()
    sp = B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.0, 0.1, 0.001)
    torch.cuda.set_device(0)
    with torch.cuda.device(0):
        assert lib.rlx_plan_grad_norm(plan._h, 1.0, None) == B.OK
        assert lib.rlx_plan_adamw(plan._h, sp, B.CLIP_FUSED, None) == B.OK
        assert lib.rlx_plan_scale_grads(plan._h, None) == B.OK
    torch.cuda.synchronize()
    assert plan.norm_read()[0] == 64.0                           # sqrt(4096 ones)
    assert lib.rlx_status_string(B.ERR_WRONG_DEVICE) == b"the plan belongs to another device than the current one"


def test_clip_rounds_twice_for_every_half_and_many_scales(O, L, host, B, torch_gpu):
    """g' = f2h(h2f(g) * scale) rounds the product to FP32 and then to FP16 (trainer.h:136-139).  A fused
    multiply-convert rounds once and differs in the last bit for about one value in 10^4, and only for
    scales with a full mantissa, so this walks every FP16 value of magnitude <= 2 under 48 different
    scales, through the scale pass and through the fused update (the check at the end makes sure that the scales met
    do tell one rounding from two)."""
    torch = torch_gpu
    pos = np.arange(0, 0x4001, dtype=np.uint32).astype(np.uint16)            # 0 .. 2.0
    vals = np.concatenate([pos, pos | 0x8000])
    n = vals.size
    specs = [L.TensorSpec("all_halves", n, L.DTYPE_F16, 0, 0)]
    mismatches_if_fused = 0
    for k in range(48):
        max_norm = 0.0123 * (1.19 ** k)
        st = host.ParamStore(specs)
        st.g16[:n].copy_(torch.from_numpy(vals.view(np.int16)).view(torch.float16))
        st.fill("p", 1, 0.0, 0.02)
        opt = host.AdamWOptimizer(st, lr=1e-3)
        torch.cuda.synchronize()
        hp = bits(st.param(0))
        norm = host.training_step(opt, max_norm, fused_clip=True)
        _, scale, _ = opt.plan.norm_read()
        assert norm > max_norm and 0 < scale < 1
        hm, hv = np.zeros(n, np.float32), np.zeros(n, np.float32)
        O.adamw_fp16(None, hp, vals.copy(), hm, hv, 1e-3, 0.9, 0.999, 1e-8, 0.01, host.bias_correction(0.9, 1),
                     host.bias_correction(0.999, 1), clip_scale=scale)
        assert np.array_equal(bits(st.state(0, "m")), hm) and np.array_equal(bits(st.state(0, "v")), hv)
        assert np.array_equal(bits(st.param(0)), hp)
        opt.plan.scale_grads()
        torch.cuda.synchronize()
        want = vals.copy()
        O.scale_half(want, scale)
        assert np.array_equal(bits(st.grad(0)), want), "scale pass, max_norm %g" % max_norm
        with np.errstate(all="ignore"):
            once = (O.h2f(vals).astype(np.float64) * np.float64(np.float32(scale))).astype(np.float16).view(np.uint16)
        mismatches_if_fused += int((once != want).sum())
    assert mismatches_if_fused >= 3, "the scales chosen would not have told one rounding from two"


def test_element_by_element_paths_with_master_fp32_and_half_precision_workspace(O, L, host, B, torch_gpu):
    """Less travelled combinations in one plan: an FP16 tensor with a master copy that starts at an odd
    element (element-by-element path), an FP32 tensor aligned to 4 but not 8 bytes, an FP16 grad-only
    buffer; norm, fused clip, gradient clearing."""
    torch = torch_gpu
    n16, n32, nw = 5003, 1001, 300
    p = torch.empty(n16 + 8, dtype=torch.float16, device="cuda:0")
    g = torch.empty(n16 + 8, dtype=torch.float16, device="cuda:0")
    m = torch.zeros(n16 + 8, dtype=torch.float32, device="cuda:0")
    v = torch.zeros(n16 + 8, dtype=torch.float32, device="cuda:0")
    w = torch.empty(n16 + 8, dtype=torch.float32, device="cuda:0")
    p32 = torch.empty(n32 + 8, dtype=torch.float32, device="cuda:0")
    g32 = torch.empty(n32 + 8, dtype=torch.float32, device="cuda:0")
    m32 = torch.zeros(n32 + 8, dtype=torch.float32, device="cuda:0")
    v32 = torch.zeros(n32 + 8, dtype=torch.float32, device="cuda:0")
    ws = torch.empty(nw + 8, dtype=torch.float16, device="cuda:0")
    B.fill_f16(p.data_ptr(), n16 + 8, 1, 0.0, 0.02)
    B.fill_f16(g.data_ptr(), n16 + 8, 2, 0.0, 5e-3)
    B.fill_f32(p32.data_ptr(), n32 + 8, 3, 1.0, 0.05)
    B.fill_f32(g32.data_ptr(), n32 + 8, 4, 0.0, 5e-3)
    B.fill_f16(ws.data_ptr(), nw + 8, 5, 0.0, 0.05)
    B.check(B.fp16_to_fp32(w.data_ptr(), p.data_ptr(), n16 + 8), "fp16_to_fp32")
    torch.cuda.synchronize()
    o16, o32, ow = 1, 1, 3
    descs = [B.TensorDesc(p.data_ptr() + 2 * o16, g.data_ptr() + 2 * o16, m.data_ptr() + 4 * o16,
                          v.data_ptr() + 4 * o16, w.data_ptr() + 4 * o16, n16, B.DTYPE_F16, 0),
             B.TensorDesc(p32.data_ptr() + 4 * o32, g32.data_ptr() + 4 * o32, m32.data_ptr() + 4 * o32,
                          v32.data_ptr() + 4 * o32, None, n32, B.DTYPE_F32, B.TENSOR_NO_DECAY),
             B.TensorDesc(None, ws.data_ptr() + 2 * ow, None, None, None, nw, B.DTYPE_F16, B.TENSOR_GRAD_ONLY)]
    hp, hg, hw = bits(p), bits(g), bits(w)
    hm, hv = np.zeros(n16 + 8, np.float32), np.zeros(n16 + 8, np.float32)
    hp32, hg32 = bits(p32), bits(g32)
    hm32, hv32 = np.zeros(n32 + 8, np.float32), np.zeros(n32 + 8, np.float32)
    hws = bits(ws)
    s16, s32, sw = slice(o16, o16 + n16), slice(o32, o32 + n32), slice(ow, ow + nw)
    plan = B.Plan(descs, 2048)
    plan.grad_norm(0.1)
    norm, scale, sum_sq = plan.norm_read()
    assert sum_sq == O.sumsq_mirror([hg[s16], hg32[s32], hws[sw]], 2048)[0] and norm > 0.1
    sp = B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.01, host.bias_correction(0.9, 1), host.bias_correction(0.999, 1))
    plan.adamw(sp, B.CLIP_FUSED | B.STEP_ZERO_GRADS)
    torch.cuda.synchronize()
    O.adamw_fp16(hw[s16], hp[s16], hg[s16], hm[s16], hv[s16], 1e-3, 0.9, 0.999, 1e-8, 0.01, sp.bias_correction1,
                 sp.bias_correction2, clip_scale=scale)
    O.adamw_fp32(hp32[s32], hg32[s32], hm32[s32], hv32[s32], 1e-3, 0.9, 0.999, 1e-8, 0.0, sp.bias_correction1,
                 sp.bias_correction2, clip_scale=scale)
    hg[s16] = 0
    hg32[s32] = 0
    hws[sw] = 0
    for got, want in ((p, hp), (g, hg), (m, hm), (v, hv), (w, hw), (p32, hp32), (g32, hg32), (m32, hm32), (v32, hv32),
                      (ws, hws)):
        assert np.array_equal(bits(got), want)              # inside as the oracle says, outside untouched
    plan.destroy()


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("RLX_RANDOM_PLAN_SEEDS", "12")))))
def test_random_plans(O, L, host, B, torch_gpu, seed):
    """Seeded random tensor lists (1 to 13 tensors, one list in four 30 to 69 so that more than 16 of them are
    frozen or grad-only, the limit up to which their gradients are cleared by range): sizes from 1 to 70,000, both dtypes, any start alignment, master copy or
    not, no-decay / frozen / grad-only flags, every chunk size, two steps with norm, fused or unfused clip
    and optional gradient clearing; every byte of every buffer (guard zones included) against the oracle."""
    torch = torch_gpu
    rng = np.random.default_rng(1000 + seed)
    count = int(rng.integers(1, 14)) if rng.integers(0, 4) else int(rng.integers(30, 70))   # many: more than 16
    chunk = int(rng.choice([512, 1024, 2048, 4096, 8192, 32768]))
    fused = bool(rng.integers(0, 2))
    zero = bool(rng.integers(0, 2))
    max_norm = float(rng.choice([0.0, 0.05, 1e6]))
    tensors, descs = [], []
    for t in range(count):
        n = int(rng.choice([rng.integers(1, 40), rng.integers(40, 3000), rng.integers(3000, 70000)]))
        f32 = bool(rng.integers(0, 4) == 0)
        flags = int(rng.choice([0, 0, B.TENSOR_NO_DECAY, B.TENSOR_FROZEN | B.TENSOR_NO_DECAY, B.TENSOR_GRAD_ONLY]))
        master = (not f32) and bool(rng.integers(0, 3) == 0) and not (flags & B.TENSOR_GRAD_ONLY)
        off = int(rng.integers(0, 9))
        tot = n + 16
        dt = torch.float32 if f32 else torch.float16
        es = 4 if f32 else 2
        d = dict(n=n, f32=f32, flags=flags, off=off, master=master)
        d["p"] = torch.empty(tot, dtype=dt, device="cuda:0")
        d["g"] = torch.empty(tot, dtype=dt, device="cuda:0")
        (B.fill_f32 if f32 else B.fill_f16)(d["p"].data_ptr(), tot, 10 * t + 1, 0.0, 0.02)
        (B.fill_f32 if f32 else B.fill_f16)(d["g"].data_ptr(), tot, 10 * t + 2, 0.0, 5e-3)
        d["m"] = torch.empty(tot, dtype=torch.float32, device="cuda:0")
        d["v"] = torch.empty(tot, dtype=torch.float32, device="cuda:0")
        frozen = bool(flags & B.TENSOR_FROZEN)
        B.fill_f32(d["m"].data_ptr(), tot, 10 * t + 3, 0.0, 0.0 if frozen else 1e-4)
        B.fill_f32(d["v"].data_ptr(), tot, 10 * t + 4, 0.0 if frozen else 1e-8, 0.0 if frozen else 1e-8, flags=1)
        d["w"] = torch.empty(tot, dtype=torch.float32, device="cuda:0") if master else None
        if master:
            B.check(B.fp16_to_fp32(d["w"].data_ptr(), d["p"].data_ptr(), tot), "fp16_to_fp32")
        grad_only = bool(flags & B.TENSOR_GRAD_ONLY)
        descs.append(B.TensorDesc(None if grad_only else d["p"].data_ptr() + es * off, d["g"].data_ptr() + es * off,
                                  None if grad_only else d["m"].data_ptr() + 4 * off,
                                  None if grad_only else d["v"].data_ptr() + 4 * off,
                                  d["w"].data_ptr() + 4 * off if master else None, n,
                                  B.DTYPE_F32 if f32 else B.DTYPE_F16, flags))
        tensors.append(d)
    torch.cuda.synchronize()
    host_side = [{k: bits(d[k]) for k in ("p", "g", "m", "v", "w") if d[k] is not None} for d in tensors]
    plan = B.Plan(descs, chunk)
    for step in (1, 2):
        scale = None
        if max_norm > 0:
            plan.grad_norm(max_norm)
            norm, scale, sum_sq = plan.norm_read()
            # frozen tensors contribute zero partials in their place of the fixed order
            mirror, parts = O.sumsq_mirror([h["g"][d["off"]: d["off"] + d["n"]] if not d["flags"] & B.TENSOR_FROZEN
                                            else np.zeros(d["n"], h["g"].dtype) for d, h in zip(tensors, host_side)],
                                           chunk)
            assert sum_sq == mirror and parts.size == plan.num_chunks
            assert scale == O.clip_scale(np.float32(sum_sq), max_norm)[0]
            if not fused:
                plan.scale_grads()
                for d, h in zip(tensors, host_side):
                    if d["flags"] & B.TENSOR_FROZEN or scale == 1.0:
                        continue
                    sl = slice(d["off"], d["off"] + d["n"])
                    (O.scale_float if d["f32"] else O.scale_half)(h["g"][sl], scale)
        bc1, bc2 = host.bias_correction(0.9, step), host.bias_correction(0.999, step)
        sp = B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.01, bc1, bc2)
        use_fused = fused and max_norm > 0
        plan.adamw(sp, (B.CLIP_FUSED if use_fused else 0) | (B.STEP_ZERO_GRADS if zero else 0))
        torch.cuda.synchronize()
        for d, h in zip(tensors, host_side):
            sl = slice(d["off"], d["off"] + d["n"])
            skip = d["flags"] & (B.TENSOR_FROZEN | B.TENSOR_GRAD_ONLY)
            if not skip:
                wd = 0.0 if d["flags"] & B.TENSOR_NO_DECAY else 0.01
                cs = scale if use_fused else None
                if d["f32"]:
                    O.adamw_fp32(h["p"][sl], h["g"][sl], h["m"][sl], h["v"][sl], 1e-3, 0.9, 0.999, 1e-8, wd, bc1, bc2,
                                 clip_scale=cs)
                else:
                    O.adamw_fp16(h["w"][sl] if d["master"] else None, h["p"][sl], h["g"][sl], h["m"][sl], h["v"][sl],
                                 1e-3, 0.9, 0.999, 1e-8, wd, bc1, bc2, clip_scale=cs)
            if zero:
                h["g"][sl] = 0
            for k in h:
                assert np.array_equal(bits(d[k]), h[k]), "seed %d step %d tensor %s buffer %s" % (seed, step, d, k)
        # fresh gradients for the second step
        for t, (d, h) in enumerate(zip(tensors, host_side)):
            (B.fill_f32 if d["f32"] else B.fill_f16)(d["g"].data_ptr(), d["n"] + 16, 100 + 10 * t + step, 0.0, 5e-3)
        torch.cuda.synchronize()
        for d, h in zip(tensors, host_side):
            h["g"] = bits(d["g"])
    plan.destroy()


@pytest.mark.gpu
def test_plan_refuses_to_launch_on_another_device(B):
    """A plan's tables belong to the device that was current when it was made."""
    import torch
    if torch.cuda.device_count() < 2:
        pytest.skip("needs two devices")
    n = 4096
    with torch.cuda.device(0):
        p = torch.zeros(n, dtype=torch.float16, device="cuda:0"); g = torch.zeros_like(p)
        m = torch.zeros(n, dtype=torch.float32, device="cuda:0"); v = torch.zeros_like(m)
        plan = B.Plan([B.TensorDesc(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), None, n, B.DTYPE_F16, 0)])
    lib = B.load()
    sp = B.StepParams(1e-3, 0.9, 0.999, 1e-8, 0.0, 0.1, 0.001)
    with torch.cuda.device(1):
        assert lib.rlx_plan_adamw(plan._h, sp, 0, None) == B.ERR_WRONG_DEVICE
        assert lib.rlx_plan_grad_norm(plan._h, 1.0, None) == B.ERR_WRONG_DEVICE
        assert lib.rlx_plan_scale_grads(plan._h, None) == B.ERR_WRONG_DEVICE
    with torch.cuda.device(0):
        assert lib.rlx_plan_adamw(plan._h, sp, 0, None) == B.OK
        torch.cuda.synchronize()
