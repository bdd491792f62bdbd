"""The callers either side of the step: scheduled learning rate, train loop with JSON-lines logging,
optimizer-state checkpoint and resume."""
import json
import math
import os

import pytest

pytestmark = pytest.mark.gpu

MINI = dict(vocab=300, hidden=64, inter=128, layers=2, q_heads=4, kv_heads=2, head_dim=16, tied=True)


def make(L, host, master):
    specs = L.qwen3_tensor_list(MINI, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
    st = host.ParamStore(specs, master=master)
    st.fill("p", 1, 0.0, 0.02)
    if master:
        st.init_master()
    return specs, st, host.AdamWOptimizer(st, lr=1e-3, chunk_elems=2048)


def snapshot(st):
    pools = [st.p16, st.p32, st.m, st.v] + ([st.master] if st.master is not None else [])
    return [t.clone() for t in pools]


@pytest.mark.parametrize("master", [False, True])
def test_checkpoint_resume_is_bit_identical(L, host, torch_gpu, tmp_path, master):
    """Three steps, save, two more steps; a fresh optimizer that loads the file and takes the same two
    steps ends with identical bits.  Weights are the model's to save: they are copied across here."""
    torch = torch_gpu
    specs, st_a, opt_a = make(L, host, master)
    for step in range(1, 4):
        st_a.fill("g", 10 + step, 0.0, 5e-3)
        host.training_step(opt_a, 0.5, fused_clip=True)
    path = str(tmp_path / "opt.state")
    if master:
        opt_a.CKPT_STAGE = 1000                  # every tensor passes through the staging buffer in several pieces
    opt_a.save_state(path)
    weights = [st_a.p16.clone(), st_a.p32.clone()]
    for step in range(4, 6):
        st_a.fill("g", 10 + step, 0.0, 5e-3)
        opt_a.set_lr(5e-4)
        host.training_step(opt_a, 0.5, fused_clip=True)
    _, st_b, opt_b = make(L, host, master)
    st_b.p16.copy_(weights[0])
    st_b.p32.copy_(weights[1])
    if master:
        opt_b.CKPT_STAGE = 333
    opt_b.load_state(path)
    assert opt_b.get_step() == 3 and abs(opt_b.lr - 1e-3) < 1e-9
    for step in range(4, 6):
        st_b.fill("g", 10 + step, 0.0, 5e-3)
        opt_b.set_lr(5e-4)
        host.training_step(opt_b, 0.5, fused_clip=True)
    torch.cuda.synchronize()
    assert opt_b.get_step() == 5
    for a, b in zip(snapshot(st_a), snapshot(st_b)):
        assert torch.equal(a, b)


def test_checkpoint_rejects_bad_files(L, host, torch_gpu, tmp_path):
    specs, st, opt = make(L, host, False)
    st.fill("g", 3, 0.0, 5e-3)
    opt.step()
    path = str(tmp_path / "opt.state")
    opt.save_state(path)
    before = snapshot(st)
    data = open(path, "rb").read()
    cases = {"foreign": b"NOTASTATE" + data[9:], "truncated": data[: len(data) // 2],
             "flipped": data[:-5] + bytes([data[-5] ^ 0x40]) + data[-4:]}
    for name, blob in cases.items():
        bad = str(tmp_path / name)
        open(bad, "wb").write(blob)
        with pytest.raises(ValueError):
            opt.load_state(bad)
        assert all(torch_gpu.equal(a, b) for a, b in zip(before, snapshot(st))), name
    _, _, other = make(L, host, True)                      # different structure: master sections expected
    with pytest.raises(ValueError):
        other.load_state(path)


# --- one optimizer-state format for the C++ class and the Python class, checked against the oracle -----------
XCFG = dict(vocab=512, hidden=128, inter=256, layers=2, q_heads=2, kv_heads=1, head_dim=128, tied=True)
XTAIL, XLR, XMAX, XSTD = 148, 1e-3, 0.5, 5e-3          # the constants of tests/cpp/ckpt_tool.cpp
XTOOL = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "ckpt_tool.bin")


class PoolWorld:
    """Python twin of the model in ckpt_tool.cpp: the same pools (every tensor a multiple of 128 elements, so
    the store's pools have no padding), the same seeds, a workspace tail that only takes part in the norm."""

    def __init__(self, L, host, torch, master=True):
        self.specs = L.qwen3_tensor_list(XCFG, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
        self.n16 = sum(s.n for s in self.specs if s.dtype == L.DTYPE_F16)
        self.n32 = sum(s.n for s in self.specs if s.dtype == L.DTYPE_F32)
        self.proj_n = self.n16 - XCFG["vocab"] * XCFG["hidden"]
        self.st = host.ParamStore(self.specs, master=master)
        assert self.st.p16.numel() == self.n16 and self.st.p32.numel() == self.n32
        self.tail = torch.zeros(XTAIL, dtype=torch.float32, device="cuda:0")
        self.host, self.L = host, L

    def optimizer(self):
        return self.host.AdamWOptimizer(self.st, lr=XLR, extra_grad_only=(self.tail,))

    def seed_weights(self, B):
        B.fill_f16(self.st.p16.data_ptr(), self.n16, 71, 0.0, 0.02)
        B.fill_f32(self.st.p32.data_ptr(), self.n32, 72, 1.0, 0.05)
        self.st.init_master()

    def step(self, B, opt, s):
        B.fill_f16(self.st.g16.data_ptr(), self.n16, 5000 + 2 * s, 0.0, XSTD)
        B.fill_f32(self.st.g32.data_ptr(), self.n32, 5001 + 2 * s, 0.0, XSTD)
        B.fill_f32(self.tail.data_ptr(), XTAIL, 5001 + 2 * s, 0.0, XSTD, first=self.n32)
        return self.host.training_step(opt, XMAX, fused_clip=False)

    def norm_groups(self, g16, g32):
        """The gradient arrays in the order of this optimizer's plan: tensor by tensor, then the tail."""
        out, o16, o32 = [], 0, 0
        for s in self.specs:
            if s.dtype == self.L.DTYPE_F16:
                out.append(g16[o16: o16 + s.n])
                o16 += s.n
            else:
                out.append(g32[o32: o32 + s.n])
                o32 += s.n
        return out + [g32[self.n32:]]


class OracleReplay:
    """The reference's order of operations on the host, from the seeded start: norm (added up in the order of
    the plan that ran the step) -> scale in place if norm > max -> three-group step."""

    def __init__(self, O, w):
        import numpy as np
        self.O, self.w, self.np = O, w, np
        self.w16 = O.fill_f16(w.n16, 71, 0.0, 0.02)
        self.w32 = O.fill_f32(w.n32, 72, 1.0, 0.05)
        self.master = O.h2f(self.w16)
        self.m16, self.v16 = np.zeros(w.n16, np.float32), np.zeros(w.n16, np.float32)
        self.m32, self.v32 = np.zeros(w.n32, np.float32), np.zeros(w.n32, np.float32)
        self.step_ = 0
        self.norms = []

    def step(self, s, cxx_order, chunk):
        O, w, np = self.O, self.w, self.np
        g16 = O.fill_f16(w.n16, 5000 + 2 * s, 0.0, XSTD)
        g32 = O.fill_f32(w.n32 + XTAIL, 5001 + 2 * s, 0.0, XSTD)
        groups = [g16[:w.proj_n], g16[w.proj_n:], g32[:w.n32], g32[w.n32:]] if cxx_order else w.norm_groups(g16, g32)
        ssq, _ = O.sumsq_mirror(groups, chunk)
        scale, norm = O.clip_scale(ssq, XMAX)
        assert norm > XMAX
        O.scale_half(g16, scale)
        O.scale_float(g32, scale)
        self.norms.append(norm)
        self.step_ = O.optimizer_step(self.master, self.w16, g16, self.m16, self.v16, w.proj_n, self.w32,
                                      np.ascontiguousarray(g32[:w.n32]), self.m32, self.v32, XLR, 0.9, 0.999, 1e-8,
                                      0.01, self.step_)


def run_tool(*args):
    import subprocess
    subprocess.run(["make", "-C", os.path.dirname(XTOOL), "-s"], check=True)      # up to date: costs nothing
    return subprocess.run([XTOOL] + [str(a) for a in args], capture_output=True, text=True, timeout=100)


def test_state_saved_by_cxx_loads_in_python_and_continues_as_the_oracle(O, B, L, host, torch_gpu, tmp_path):
    """ckpt_tool (C++ AdamWOptimizer) takes 3 steps and saves; the Python AdamWOptimizer loads that file and
    takes steps 4 and 5; weights, master copy and moments equal the oracle's five steps from the seeded start."""
    import numpy as np
    from util import bits
    torch = torch_gpu
    res = run_tool("save", tmp_path, 3)
    assert res.returncode == 0, res.stdout + res.stderr
    w = PoolWorld(L, host, torch)
    w.st.p16.copy_(torch.from_numpy(np.fromfile(tmp_path / "w16.bin", dtype=np.int16)).view(torch.float16))
    w.st.p32.copy_(torch.from_numpy(np.fromfile(tmp_path / "w32.bin", dtype=np.float32)))
    opt = w.optimizer()
    opt.load_state(str(tmp_path / "opt.state"))
    assert opt.get_step() == 3
    got_norms = [w.step(B, opt, s) for s in (4, 5)]
    torch.cuda.synchronize()
    rep = OracleReplay(O, w)
    for s in (1, 2, 3):
        rep.step(s, cxx_order=True, chunk=8192)
    cxx_norms = [float(line.split()[3]) for line in res.stdout.splitlines() if line.startswith("step ")]
    assert [np.float32(x) for x in cxx_norms] == [np.float32(x) for x in rep.norms]
    for s in (4, 5):
        rep.step(s, cxx_order=False, chunk=opt.plan.chunk_elems)
    assert [np.float32(x) for x in got_norms] == [np.float32(x) for x in rep.norms[3:]]
    st = w.st
    assert np.array_equal(bits(st.p16), rep.w16) and np.array_equal(bits(st.p32).view(np.uint32), rep.w32.view(np.uint32))
    assert np.array_equal(bits(st.master[:w.n16]).view(np.uint32), rep.master.view(np.uint32))
    for got, want in ((st.m[:w.n16], rep.m16), (st.v[:w.n16], rep.v16), (st.m[w.n16:], rep.m32), (st.v[w.n16:], rep.v32)):
        assert np.array_equal(bits(got).view(np.uint32), want.view(np.uint32))
    # the same file does not fit an optimizer without a master copy, and the error says so
    other = PoolWorld(L, host, torch, master=False).optimizer()
    with pytest.raises(ValueError, match="different layout"):
        other.load_state(str(tmp_path / "opt.state"))


def test_state_saved_by_python_loads_in_cxx_and_continues_as_the_oracle(O, B, L, host, torch_gpu, tmp_path):
    """The Python AdamWOptimizer takes 3 steps and saves; ckpt_tool loads that file into the C++ class and takes
    steps 4 and 5; what it ends with equals the oracle's five steps.  A damaged copy of the file is refused."""
    import numpy as np
    from util import bits
    torch = torch_gpu
    w = PoolWorld(L, host, torch)
    w.seed_weights(B)
    opt = w.optimizer()
    for s in (1, 2, 3):
        w.step(B, opt, s)
    torch.cuda.synchronize()
    opt.save_state(str(tmp_path / "opt.state"))
    bits(w.st.p16).tofile(tmp_path / "w16.bin")
    bits(w.st.p32).tofile(tmp_path / "w32.bin")
    res = run_tool("load", tmp_path, 3, 2)
    assert res.returncode == 0, res.stdout + res.stderr
    rep = OracleReplay(O, w)
    for s in (1, 2, 3):
        rep.step(s, cxx_order=False, chunk=opt.plan.chunk_elems)
    for s in (4, 5):
        rep.step(s, cxx_order=True, chunk=8192)
    cxx_norms = [float(line.split()[3]) for line in res.stdout.splitlines() if line.startswith("step ")]
    assert [np.float32(x) for x in cxx_norms] == [np.float32(x) for x in rep.norms[3:]]
    assert np.array_equal(np.fromfile(tmp_path / "out_w16.bin", dtype=np.uint16), rep.w16)
    for name, want in (("w32", rep.w32), ("master", rep.master), ("m16", rep.m16), ("v16", rep.v16),
                       ("m32", rep.m32), ("v32", rep.v32)):
        assert np.array_equal(np.fromfile(tmp_path / ("out_%s.bin" % name), dtype=np.uint32), want.view(np.uint32)), name
    # a flipped data bit, a cut file and a foreign file are refused by the C++ loader (exit code 3)
    good = open(tmp_path / "opt.state", "rb").read()
    for blob in (good[:-5] + bytes([good[-5] ^ 0x40]) + good[-4:], good[: len(good) // 2], b"RLXOPT01" + good[8:]):
        open(tmp_path / "opt.state", "wb").write(blob)
        assert run_tool("load", tmp_path, 3, 1).returncode == 3


def test_train_loop_logs_jsonl(O, L, host, torch_gpu, tmp_path, capsys):
    """Cosine schedule with warm-up drives set_lr; every second step one JSON line with the window means of
    loss, lr, grad_norm, step_ms, tok_per_sec (the keys of include/training/trainer.h:208-212).
    The loop is pinned to the oracle: the reference logs the pre-clip norm that clip_grad_norm_ returns and its
    weights follow from set_lr + clip + step (trainer.h:183-225, 288, 351), so the oracle replays the eight steps
    on the host (scheduler's rate -> norm in the plan's order -> clip rule -> step) and every logged window mean
    of grad_norm, the state file written at save_steps and the parameters and moments after the loop must be
    the oracle's, bit for bit."""
    import numpy as np
    from test_gpu_plan import compare, host_copy, oracle_step
    from util import HYPER, bits
    torch = torch_gpu
    specs, st, opt = make(L, host, False)
    sched = host.LRScheduler()
    sched.init_cosine(1e-3, 1e-4, 2, 8)
    log_dir = str(tmp_path / "run")
    logger = host.Logger(log_dir)
    losses, oracle_norms = [], []
    torch.cuda.synchronize()
    hs = host_copy(st)
    state_path = str(tmp_path / "opt.state")

    def produce(step):
        if step == 4:       # the loop has just saved the state of step 4: it reloads to the oracle's state
            _, st_b, opt_b = make(L, host, False)
            opt_b.load_state(state_path)
            assert opt_b.get_step() == 4 and opt_b.lr == sched.get_lr(3)
            for i, h in enumerate(hs):
                assert np.array_equal(bits(st_b.state(i, "m")), h["m"]) and np.array_equal(bits(st_b.state(i, "v")), h["v"])
        st.fill("g", 100 + step, 0.0, 5e-3)
        torch.cuda.synchronize()
        for i, h in enumerate(hs):
            h["g"] = bits(st.grad(i))
        ssq, _ = O.sumsq_mirror([h["g"] for h in hs], opt.plan.chunk_elems)
        scale, norm = O.clip_scale(np.float32(ssq), 0.5)
        oracle_step(O, L, specs, hs, step + 1, dict(HYPER, lr=sched.get_lr(step)), clip_scale=scale)
        oracle_norms.append(np.float32(norm))
        losses.append(3.0 / (1 + step))
        return losses[-1]

    done = host.train_loop(opt, sched, logger, produce, total_steps=8, max_grad_norm=0.5, logging_steps=2,
                           save_steps=4, save_path=state_path, tokens_per_step=4096)
    logger.close()
    assert done == 8 and opt.get_step() == 8 and os.path.exists(state_path)
    torch.cuda.synchronize()
    assert compare(st, hs, "after the loop") == 0
    rows = [json.loads(l) for l in open(os.path.join(log_dir, "train_log.jsonl"))]
    assert [r["step"] for r in rows] == [2, 4, 6, 8]
    assert all(sorted(r) == ["grad_norm", "loss", "lr", "step", "step_ms", "tok_per_sec"] for r in rows)
    for k, r in enumerate(rows):
        s0, s1 = 2 * k, 2 * k + 1
        assert abs(r["loss"] - (losses[s0] + losses[s1]) / 2) < 1e-6
        assert abs(r["lr"] - (sched.get_lr(s0) + sched.get_lr(s1)) / 2) < 1e-9
        want = np.float32(np.float32(np.float32(0.0) + oracle_norms[s0]) + oracle_norms[s1]) / np.float32(2)   # FP32 window mean
        assert abs(r["grad_norm"] - float(want)) <= 1e-7 * float(want) and r["grad_norm"] == float(want)
        assert oracle_norms[s0] > 0.5 and r["step_ms"] > 0 and r["tok_per_sec"] > 0
    assert abs(opt.lr - sched.get_lr(7)) < 1e-12
    assert logger.last("loss") == rows[-1]["loss"] and math.isnan(logger.last("nope")) and len(logger.history()) == 4
    assert "[step 8]" in capsys.readouterr().out
    # a restart appends to the same file
    logger2 = host.Logger(log_dir)
    logger2.log(9, {"loss": 1.0, "lr": 1e-4})
    logger2.commit(9)
    logger2.close()
    assert len(open(os.path.join(log_dir, "train_log.jsonl")).readlines()) == 5


def test_steps_reduce_a_loss(L, host, torch_gpu):
    """The last case of the reference's own test (tests/test_adamw.cu:453-501: five steps at lr=1e-4 reduce
    the model's NLL), on a loss that needs no model: 0.5 * |p - target|^2 with its exact gradient."""
    torch = torch_gpu
    specs = [L.TensorSpec("w", 50_000, L.DTYPE_F16, 0, 0), L.TensorSpec("n", 500, L.DTYPE_F32, L.NO_DECAY, 0)]
    st = host.ParamStore(specs, master=True)
    st.fill("p", 1, 0.0, 0.5)
    st.init_master()
    target16 = torch.full((50_000,), 0.25, dtype=torch.float16, device="cuda:0")
    target32 = torch.full((500,), -0.5, dtype=torch.float32, device="cuda:0")
    opt = host.AdamWOptimizer(st, lr=1e-2, weight_decay=0.0)

    def loss_and_grads():
        d16 = st.param(0).float() - target16.float()
        d32 = st.param(1) - target32
        st.grad(0).copy_(d16.half())
        st.grad(1).copy_(d32)
        return 0.5 * (d16.pow(2).sum() + d32.pow(2).sum()).item()

    losses = []
    for _ in range(5):
        losses.append(loss_and_grads())
        host.training_step(opt, 1.0, fused_clip=True)
    losses.append(loss_and_grads())
    assert all(b < a for a, b in zip(losses, losses[1:])), losses
    assert opt.get_step() == 5


def test_plans_can_be_created_and_destroyed_many_times(L, host, B, torch_gpu):
    """A plan owns device tables, a workspace and pinned memory: 300 create / use / destroy rounds leave the
    device's free memory where it was."""
    torch = torch_gpu
    specs = L.qwen3_tensor_list(MINI)
    st = host.ParamStore(specs)
    st.fill("g", 1, 0.0, 1e-3)
    descs = st.descs()
    torch.cuda.synchronize()
    p = B.Plan(descs, 2048)
    p.grad_norm(1.0)
    first = p.norm_read()
    p.destroy()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(300):
        p = B.Plan(descs, 2048)
        p.grad_norm(1.0)
        assert p.norm_read() == first
        p.destroy()
    free1, _ = torch.cuda.mem_get_info()
    assert abs(free0 - free1) < 8 * 2 ** 20
    p.destroy()                                   # a second destroy of the wrapper is harmless


def test_two_host_threads_with_their_own_plans_and_streams(O, L, host, B, torch_gpu):
    """Two host threads step two optimizers on two streams at the same time; each result equals the
    oracle's.  (One plan is not shared between threads: that is documented as unsupported.)"""
    import threading
    import numpy as np
    from util import bits
    torch = torch_gpu
    specs = [L.TensorSpec("w", 300_000, L.DTYPE_F16, 0, 0), L.TensorSpec("n", 999, L.DTYPE_F32, L.NO_DECAY, 0)]
    stores, opts, streams = [], [], [torch.cuda.Stream(), torch.cuda.Stream()]
    for k in range(2):
        s = host.ParamStore(specs)
        s.fill("p", 1 + k, 0.0, 0.02)
        s.fill("g", 3 + k, 0.0, 5e-3)
        stores.append(s)
        opts.append(host.AdamWOptimizer(s, lr=1e-3 * (k + 1)))
    torch.cuda.synchronize()
    before = [[(bits(s.param(i)), bits(s.grad(i))) for i in range(2)] for s in stores]
    norms, errors = [None, None], []

    def work(k):
        try:
            with torch.cuda.stream(streams[k]):
                for _ in range(20):
                    norms[k] = host.training_step(opts[k], 0.5, fused_clip=True)
                streams[k].synchronize()
        except Exception as exc:      # pragma: no cover
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for k in range(2):
        hs = [dict(p=before[k][i][0], g=before[k][i][1], m=np.zeros(specs[i].n, np.float32),
                   v=np.zeros(specs[i].n, np.float32)) for i in range(2)]
        ssq, _ = O.sumsq_mirror([h["g"] for h in hs], opts[k].plan.chunk_elems)
        scale, norm = O.clip_scale(np.float32(ssq), 0.5)
        assert norms[k] == norm
        for step in range(1, 21):
            bc1, bc2 = host.bias_correction(0.9, step), host.bias_correction(0.999, step)
            O.adamw_fp16(None, hs[0]["p"], hs[0]["g"], hs[0]["m"], hs[0]["v"], 1e-3 * (k + 1), 0.9, 0.999, 1e-8, 0.01,
                         bc1, bc2, clip_scale=scale)
            O.adamw_fp32(hs[1]["p"], hs[1]["g"], hs[1]["m"], hs[1]["v"], 1e-3 * (k + 1), 0.9, 0.999, 1e-8, 0.0,
                         bc1, bc2, clip_scale=scale)
        for i in range(2):
            assert np.array_equal(bits(stores[k].param(i)), hs[i]["p"])
            assert np.array_equal(bits(stores[k].state(i, "v")), hs[i]["v"])


@pytest.mark.parametrize("fused", [False, True])
def test_accumulation_step_follows_the_reference_order(O, L, host, B, torch_gpu, fused):
    """training_step of the reference (include/training/trainer.h:231-289) with three micro-batches: clear
    the pools, scale each micro-batch's loss gradient by 1/3 before its backward pass adds into the pools,
    clear the frozen embedding's gradients, clip, step.  The backward pass here is a stand-in made of
    element-wise operations only (so that host and device agree exactly); everything else is the library,
    checked against numpy + the oracle in the same order."""
    import numpy as np
    from util import HYPER, bits
    from test_gpu_plan import compare, host_copy, oracle_step
    torch = torch_gpu
    specs, st, opt = make(L, host, master=False)
    emb = [i for i, s in enumerate(specs) if s.name == "embed_tokens"][0]
    acc, T = 3, 37
    loss_grad = torch.empty(T, dtype=torch.float32, device="cuda:0")
    st.fill("g", 999, 0.0, 1.0)                       # stale gradients that the step must clear first
    torch.cuda.synchronize()
    hs = host_copy(st)
    for h in hs:
        h["g"][...] = 0
    scale = np.float32(1.0) / np.float32(acc)
    base16 = [torch.empty_like(st.g16), None]
    base32 = torch.empty_like(st.g32)

    def micro_batch(k, scale_loss_grad):
        B.fill_f32(loss_grad.data_ptr(), T, 500 + k, 2.0, 0.5)          # "compute_loss"
        lg_h = O.fill_f32(T, 500 + k, 2.0, 0.5)
        scale_loss_grad()
        lg_h = lg_h * scale
        # "backward": pools += seeded pattern * loss_grad[0], element-wise
        B.fill_f16(base16[0].data_ptr(), base16[0].numel(), 600 + k, 0.0, 2e-3)
        B.fill_f32(base32.data_ptr(), base32.numel(), 700 + k, 0.0, 2e-3)
        f = loss_grad[0]
        st.g16.add_((base16[0].float() * f).half())
        st.g32.add_(base32 * f)
        b16 = O.h2f(O.fill_f16(base16[0].numel(), 600 + k, 0.0, 2e-3))
        b32 = O.fill_f32(base32.numel(), 700 + k, 0.0, 2e-3)
        for i, s in enumerate(specs):
            lo = st.off_pg[i]
            if s.dtype == L.DTYPE_F16:
                add = (b16[lo:lo + s.n] * lg_h[0]).astype(np.float16)
                cur = hs[i]["g"].view(np.float16)
                hs[i]["g"] = (cur.astype(np.float32) + add.astype(np.float32)).astype(np.float16).view(np.uint16)
            else:
                hs[i]["g"] = (hs[i]["g"] + b32[lo:lo + s.n] * lg_h[0]).astype(np.float32)
        return float(k + 1)

    loss, norm = host.accumulation_step(opt, micro_batch, acc, 0.05, loss_grad=loss_grad, fused_clip=fused,
                                        freeze=[st.grad(emb)])
    torch.cuda.synchronize()
    assert loss == 2.0
    hs[emb]["g"][...] = 0
    sq = sum(float((O.h2f(h["g"]).astype(np.float64) ** 2).sum()) if h["g"].dtype == np.uint16
             else float((h["g"].astype(np.float64) ** 2).sum()) for h in hs)
    assert abs(norm - math.sqrt(sq)) <= 1e-5 * math.sqrt(sq) and norm > 0.05
    _, s_dev, _ = opt.plan.norm_read()
    assert not st.grad(emb).any().item()
    if not fused:                                     # the scale pass rewrote the gradients: compare them too
        for i, h in enumerate(hs):
            exp = h["g"].copy()
            (O.scale_half if exp.dtype == np.uint16 else O.scale_float)(exp, s_dev)
            assert np.array_equal(bits(st.grad(i)), exp), "scaled gradients, tensor %d" % i
    oracle_step(O, L, specs, hs, 1, dict(HYPER, lr=1e-3), clip_scale=s_dev)
    assert compare(st, hs, "accumulation step") == 0
