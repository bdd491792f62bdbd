"""Full-size workloads on the GPU: Qwen3-0.6B (update; norm + clip) and Qwen3-8B (98 GB resident).
The oracle replays sampled slices (the update is elementwise, so a slice is checked exactly as
the whole would be); whole-tensor properties (determinism, fused == unfused, norm stability) are
checked on the device."""
import numpy as np
import pytest

from util import bits, read_device

pytestmark = pytest.mark.gpu

HY = dict(lr=1e-5, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)
THR90 = int(0.9 * 2 ** 32)


def sample_slices(specs, rng, per_tensor=2, width=5000):
    """(tensor, lo, n): heads, tails and random interiors of the big tensors, all small tensors."""
    out = []
    for i, s in enumerate(specs):
        if s.n <= 4096:
            if i % 16 == 0 or i == len(specs) - 1:
                out.append((i, 0, s.n))
            continue
        if i % 23 != 0 and s.n < 100_000_000:
            continue
        w = min(width, s.n)
        out.append((i, 0, w))
        out.append((i, s.n - w, w))
        for _ in range(per_tensor):
            out.append((i, int(rng.integers(0, s.n - w)), w))
    return out


def grab(store, which, i, lo, n):
    t = store.param(i) if which == "p" else store.grad(i) if which == "g" else store.state(i, which)
    return bits(t[lo: lo + n])


def test_qwen3_0_6b_hundred_steps_sampled(O, L, host, torch_gpu):
    """310 tensors / 596,049,920 parameters; gradients ~N(0,1e-4) with 90% of the embedding rows
    zero, fresh every step; 100 steps; the oracle replays every step on the sampled slices."""
    torch = torch_gpu
    specs = L.qwen3_tensor_list(L.QWEN3_0_6B)
    emb = [i for i, s in enumerate(specs) if s.name == "embed_tokens"][0]
    st = host.ParamStore(specs)
    st.fill("p", 0x5EED0001, 0.0, 0.02)
    opt = host.AdamWOptimizer(st, lr=HY["lr"])
    assert opt.plan.num_elements == 596_049_920 and opt.plan.chunk_elems == 8192
    samp = sample_slices(specs, np.random.default_rng(1))
    assert any(i == emb for i, _, _ in samp)
    torch.cuda.synchronize()
    ref = [dict(p=grab(st, "p", i, lo, n), m=np.zeros(n, np.float32), v=np.zeros(n, np.float32))
           for i, lo, n in samp]
    for step in range(1, 101):
        seed = 0x6EAD0001 + step
        st.fill("g", seed, 0.0, 1e-4, zero_row_frac=0.9, only=("embed_tokens",))
        opt.step()
        bc1, bc2 = host.bias_correction(HY["beta1"], step), host.bias_correction(HY["beta2"], step)
        for (i, lo, n), r in zip(samp, ref):
            g = O.fill_f16(n, L._hash64(seed, i), 0.0, 1e-4, first=lo,
                           row_len=specs[i].row_len if i == emb else 0, zero_rows_below=THR90 if i == emb else 0)
            O.adamw_fp16(None, r["p"], g, r["m"], r["v"], HY["lr"], HY["beta1"], HY["beta2"], HY["eps"], HY["wd"],
                         bc1, bc2)
    torch.cuda.synchronize()
    assert opt.get_step() == 100
    for (i, lo, n), r in zip(samp, ref):
        for k in ("p", "m", "v"):
            assert np.array_equal(grab(st, k, i, lo, n), r[k]), "tensor %d [%d:+%d] %s" % (i, lo, n, k)
    # zero gradient rows of the embedding: moments stay zero, weights only decay
    e_m = st.state(emb, "m").view(151936, 1024)
    zero_rows = (~e_m.any(dim=1)).float().mean().item()
    assert zero_rows < 0.01           # over 100 steps nearly every row has been touched at least once


def test_qwen3_0_6b_norm_clip_fused_vs_unfused(O, L, host, torch_gpu):
    """Gradients ~N(0,5e-3): norm about 122, clipping to 1.0 active.  Norm: 1e-5 against FP64 on the
    host, bit-identical to the restated device order, the same bits on ten runs.  The fused step
    equals scale pass + plain step on every element; sampled slices equal the oracle."""
    torch = torch_gpu
    specs = L.qwen3_tensor_list(L.QWEN3_0_6B)
    stores = []
    for _ in range(2):
        st = host.ParamStore(specs)
        st.fill("p", 0x5EED0002, 0.0, 0.02)
        st.fill("m", 0x5EED0003, 0.0, 1e-4)
        st.fill("v", 0x5EED0004, 1e-8, 1e-8, flags=1)
        st.fill("g", 0x5EED0005, 0.0, 5e-3)
        stores.append(st)
    opts = [host.AdamWOptimizer(s, lr=HY["lr"]) for s in stores]
    for o in opts:
        o.step_ = 99
    torch.cuda.synchronize()
    samp = sample_slices(specs, np.random.default_rng(2))
    ref = [{k: grab(stores[0], k, i, lo, n) for k in "pgmv"} for i, lo, n in samp]
    seen = set()
    for _ in range(10):
        opts[0].plan.grad_norm(1.0)
        seen.add(opts[0].plan.norm_read())
    assert len(seen) == 1
    norm, scale, sum_sq = seen.pop()
    g_host = bits(stores[0].g16)               # every tensor size is a multiple of 128: no padding in between
    assert g_host.size == 596_049_920
    truth = O.sum_sq_half(g_host)
    assert abs(sum_sq - truth) <= 1e-5 * truth
    assert abs(norm - np.sqrt(truth)) <= 1e-5 * np.sqrt(truth) and 100 < norm < 150
    offs = np.cumsum([0] + [s.n for s in specs])
    mirror, _ = O.sumsq_mirror([g_host[offs[i]: offs[i + 1]] for i in range(len(specs))], 8192)
    assert sum_sq == mirror
    assert scale == O.clip_scale(np.float32(sum_sq), 1.0)[0]
    del g_host
    n0 = opts[0].clip_grad_norm_(1.0)          # scales gradients in place
    opts[0].step()
    n1 = host.training_step(opts[1], 1.0, fused_clip=True)
    torch.cuda.synchronize()
    assert n0 == n1 == norm and opts[0].get_step() == opts[1].get_step() == 100
    for a, b in ((stores[0].p16, stores[1].p16), (stores[0].m, stores[1].m), (stores[0].v, stores[1].v)):
        assert torch.equal(a, b), "fused and unfused steps differ"
    post = stores[0].g16.double().pow(2).sum().sqrt().item()
    assert abs(post - 1.0) < 2e-3               # clipped gradients have norm ~ max_norm (FP16 re-rounding)
    bc1, bc2 = host.bias_correction(HY["beta1"], 100), host.bias_correction(HY["beta2"], 100)
    for (i, lo, n), r in zip(samp, ref):
        O.adamw_fp16(None, r["p"], r["g"], r["m"], r["v"], HY["lr"], HY["beta1"], HY["beta2"], HY["eps"], HY["wd"],
                     bc1, bc2, clip_scale=scale)
        for k in ("p", "m", "v"):
            assert np.array_equal(grab(stores[1], k, i, lo, n), r[k]), "tensor %d [%d:+%d] %s" % (i, lo, n, k)


def test_qwen3_8b_resident(O, L, host, torch_gpu):
    """399 tensors / 8.19e9 parameters, 98 GB resident: 64-bit indexing, several launches per step.
    Moments are seeded directly (m ~N(0,1e-4), v = 1e-8 (1+|z|)) for a step at t = 1000; gradients
    ~N(0,1e-4); clip at 1.0 (norm about 9).  Norm against torch's FP64 on the device (an independent
    reduction); sampled slices against the oracle, including elements beyond index 2^32."""
    torch = torch_gpu
    free, _ = torch.cuda.mem_get_info()
    if free < 110 * 2 ** 30:
        pytest.skip("needs 110 GB of free device memory")
    specs = L.qwen3_tensor_list(L.QWEN3_8B)
    st = host.ParamStore(specs, zero_state=False)
    st.fill("p", 0x5EED0010, 0.0, 0.02)
    st.fill("g", 0x5EED0011, 0.0, 1e-4)
    st.fill("m", 0x5EED0012, 0.0, 1e-4)
    st.fill("v", 0x5EED0013, 1e-8, 1e-8, flags=1)
    opt = host.AdamWOptimizer(st, lr=HY["lr"])
    opt.step_ = 999
    assert opt.plan.num_elements == 8_190_735_360 and opt.plan.chunk_elems == 32768 and opt.plan.num_chunks > 240_000
    torch.cuda.synchronize()
    samp = sample_slices(specs, np.random.default_rng(3), per_tensor=3)
    assert any(st.off[i] + lo > 2 ** 32 for i, lo, _ in samp) and len(samp) > 60
    ref = [{k: grab(st, k, i, lo, n) for k in "pgmv"} for i, lo, n in samp]
    for (i, lo, n), r in zip(samp[:8], ref[:8]):       # device generator == host generator at large offsets
        assert np.array_equal(r["g"], O.fill_f16(n, L._hash64(0x5EED0011, i), 0.0, 1e-4, first=lo))
    tot = 0.0
    step_elems = 1 << 28
    for lo in range(0, st.g16.numel(), step_elems):
        tot += st.g16[lo: lo + step_elems].double().pow(2).sum().item()
    norm = host.training_step(opt, 1.0, fused_clip=True)
    torch.cuda.synchronize()
    n2, scale, sum_sq = opt.plan.norm_read()
    assert n2 == norm and abs(sum_sq - tot) <= 1e-5 * tot and 8.5 < norm < 9.6
    assert scale == O.clip_scale(np.float32(sum_sq), 1.0)[0] and opt.get_step() == 1000
    bc1, bc2 = host.bias_correction(HY["beta1"], 1000), host.bias_correction(HY["beta2"], 1000)
    for (i, lo, n), r in zip(samp, ref):
        O.adamw_fp16(None, r["p"], r["g"], r["m"], r["v"], HY["lr"], HY["beta1"], HY["beta2"], HY["eps"], HY["wd"],
                     bc1, bc2, clip_scale=scale)
        for k in ("p", "m", "v"):
            assert np.array_equal(grab(st, k, i, lo, n), r[k]), "tensor %d [%d:+%d] %s" % (i, lo, n, k)
        assert np.array_equal(grab(st, "g", i, lo, n), r["g"])
    # a second, identical run of the norm gives the same bits
    opt.plan.grad_norm(1.0)
    assert opt.plan.norm_read() == (n2, scale, sum_sq)
    # the million per-chunk partials: their fixed-order sum is the result, and sampled chunks (random ones, the
    # last and possibly short chunk of every tensor, chunks whose elements lie beyond index 2^32) equal the
    # restated reduction order on gradients regenerated on the host
    chunk = opt.plan.chunk_elems
    parts = read_device(opt.plan.partials_ptr, 8 * opt.plan.num_chunks).view(np.float64)
    assert O.sumsq_mirror_final(parts) == sum_sq
    first_chunk = np.cumsum([0] + [-(-s.n // chunk) for s in specs])
    assert first_chunk[-1] == opt.plan.num_chunks
    rng = np.random.default_rng(11)
    picks = [(i, int(first_chunk[i + 1] - first_chunk[i]) - 1) for i in range(len(specs))]
    picks += [(int(i), int(rng.integers(0, first_chunk[i + 1] - first_chunk[i]))) for i in rng.integers(0, len(specs), 200)]
    beyond = 0
    for i, c in picks:
        lo = c * chunk
        n = min(chunk, specs[i].n - lo)
        beyond += st.off[i] + lo > 2 ** 32
        g = O.fill_f16(n, L._hash64(0x5EED0011, i), 0.0, 1e-4, first=lo)
        _, one = O.sumsq_mirror([g], chunk)
        got = parts[first_chunk[i] + c]
        assert one.size == 1 and one.view(np.uint64)[0] == np.float64(got).view(np.uint64), "tensor %d chunk %d" % (i, c)
    assert beyond > 100


def test_single_tensor_beyond_int32(O, B, host, torch_gpu):
    """One flat tensor of 2^31 + 1001 parameters through the operator API (the reference's `int n` cannot
    express it): several launches, byte offsets beyond 2^32, an odd tail.  Slices at the start, across the
    2^31 boundary and at the very end are replayed by the oracle."""
    torch = torch_gpu
    n = 2 ** 31 + 1001
    free, _ = torch.cuda.mem_get_info()
    if free < 30 * 2 ** 30:
        pytest.skip("needs 30 GB of free device memory")
    p = torch.empty(n, dtype=torch.float16, device="cuda:0")
    g = torch.empty(n, dtype=torch.float16, device="cuda:0")
    m = torch.empty(n, dtype=torch.float32, device="cuda:0")
    v = torch.empty(n, dtype=torch.float32, device="cuda:0")
    B.fill_f16(p.data_ptr(), n, 1, 0.0, 0.02)
    B.fill_f16(g.data_ptr(), n, 2, 0.0, 1e-3)
    B.fill_f32(m.data_ptr(), n, 3, 0.0, 1e-4)
    B.fill_f32(v.data_ptr(), n, 4, 1e-8, 1e-8, flags=1)
    torch.cuda.synchronize()
    slices = [(0, 3000), (2 ** 31 - 1500, 2400), (n - 1001 - 300, 1301), (123456789 * 8 + 3, 2000)]
    ref = [dict(p=bits(p[lo: lo + k]), g=bits(g[lo: lo + k]), m=bits(m[lo: lo + k]), v=bits(v[lo: lo + k]))
           for lo, k in slices]
    assert np.array_equal(ref[1]["g"], O.fill_f16(2400, 2, 0.0, 1e-3, first=2 ** 31 - 1500))
    bc1, bc2 = host.bias_correction(0.9, 7), host.bias_correction(0.999, 7)
    assert B.adamw_fp16(None, p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), n, 1e-4, 0.9, 0.999, 1e-8,
                        0.01, bc1, bc2) == B.OK
    torch.cuda.synchronize()
    for (lo, k), r in zip(slices, ref):
        O.adamw_fp16(None, r["p"], r["g"], r["m"], r["v"], 1e-4, 0.9, 0.999, 1e-8, 0.01, bc1, bc2)
        assert np.array_equal(bits(p[lo: lo + k]), r["p"]), lo
        assert np.array_equal(bits(m[lo: lo + k]), r["m"]) and np.array_equal(bits(v[lo: lo + k]), r["v"]), lo
