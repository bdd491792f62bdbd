#!/usr/bin/env python3
"""Benchmark of the AdamW step on one MI355X.

Headline workload (N=1): the Qwen3-0.6B parameter set as a 310-tensor list, FP16 parameters and
gradients, FP32 moments, no master copy; moments pre-populated by 99 seeded steps; timed steps
are steps 100, 101, ... over resident inputs: one multi-tensor update launch each (22 bytes per
parameter: read p, g, m, v; write p, m, v).  The same list with the norm + fused-clip step is
timed too and reported under "clip_step".

The default run also measures the other configurations (one flat tensor of 1,048,576 parameters, the
4,096-tensor ragged list beside one flat tensor of the same element count, the Qwen3-8B list, and
Qwen3-0.6B in the reference's 28-byte layout with an FP32 master copy) and reports them under "configs":
update, norm, norm + fused-clip update, each in ms and GB/s (seeded state, no oracle replay: the GPU tests
hold the parity of these configurations).  --configs none skips them (short profiler runs).

Prints ONE JSON line.  The CPU oracle is used here only as the checker of a sample and as the
timed CPU baseline: the oracle's threaded step on a slice of the embedding's state ("cpu_baseline") and on every
configuration at its own size ("cpu_baseline.configs": all 310 tensors of Qwen3-0.6B, the flat tensor, the 4,096-tensor
list as one split / as a loop of one call per tensor / beside one flat tensor, a 1e9-parameter slice of Qwen3-8B),
with 16 threads and with one; its inputs are copied to the host before the timed GPU steps and every CPU pass starts
from that saved state.

Beside the eager legs, "clip_step" holds the parts of the clip step in the same run (plain update on dense gradients,
fused-clip update alone, norm) and every configuration holds "graph_clip_step_ms": norm + scheduled fused-clip update
recorded once as a HIP graph and replayed.

--workload selects one of the other configurations as the line's subject instead (flat-1m,
qwen3-0.6b-master, ragged, qwen3-8b): the same kind of line with fewer legs.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBPS = 8000.0
BYTES_UPDATE = 22          # per parameter: R p2 g2 m4 v4, W p2 m4 v4
BYTES_NORM = 2             # per parameter: R g2
SEED_P, SEED_G = 0x5EED0001, 0x6EAD0001
STORAGE = "fp16 params and grads, fp32 moments; arithmetic in fp32"
SECONDARY = ("flat-1m", "ragged", "qwen3-0.6b-master", "qwen3-8b")


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def host_cpus():
    """What this process may use: logical CPUs, the affinity mask, and the cgroup's quota if there is one."""
    info = {"nproc": os.cpu_count() or 1}
    try:
        info["affinity"] = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        info["affinity"] = info["nproc"]
    try:
        quota, period = open("/sys/fs/cgroup/cpu.max").read().split()
        info["cgroup_cpus"] = None if quota == "max" else float(quota) / float(period)
    except (OSError, ValueError):
        info["cgroup_cpus"] = None
    return info


def cpu_baseline(O, host, sample, g_clip, hyper, step, seconds=5.0):
    """The oracle's threaded FP16 step on a slice of the same workload, on the host's cores: the update alone
    (the configuration of the headline), and norm + clip + update with the larger gradients of the clip
    configuration (FP64 sum of squares, sqrt, scale = max/(norm+1e-6f) iff norm > max, then the update with
    the scaled and re-rounded gradients), with 16 threads (the CPU share of a one-GPU box) and with every core the
    process may use.
    Every timed pass starts from the saved state of step 99 (restored outside the timed region): the port's speed
    depends on the values (this host's divider is data dependent), and repeating one step in place on fixed
    gradients drives the first moments towards zero and the step from 12.4 to 4.9 ms per Mi parameters.  Each leg
    is repeated until about `seconds` of wall time have passed."""
    p0, g, m0, v0 = sample
    cpus = host_cpus()
    t16 = min(16, cpus["affinity"])
    t_all = cpus["affinity"]
    bc1, bc2 = host.bias_correction(hyper["beta1"], step), host.bias_correction(hyper["beta2"], step)
    args = (hyper["lr"], hyper["beta1"], hyper["beta2"], hyper["eps"], hyper["wd"], bc1, bc2)

    def rate(n, grad, max_norm, threads, budget):
        """params/s over passes that each start from the saved state; (rate, passes, timed seconds)."""
        p, m, v = p0[:n].copy(), m0[:n].copy(), v0[:n].copy()
        gg = grad[:n]
        O.step_fp16_threaded(None, p, gg, m, v, *args, max_norm, threads)        # touch pages, warm caches
        reps, timed, wall0 = 0, 0.0, time.perf_counter()
        while True:
            p[:], m[:], v[:] = p0[:n], m0[:n], v0[:n]
            t0 = time.perf_counter()
            O.step_fp16_threaded(None, p, gg, m, v, *args, max_norm, threads)
            timed += time.perf_counter() - t0
            reps += 1
            if time.perf_counter() - wall0 >= budget or reps >= 200:
                break
        return n * reps / timed, reps, timed

    n_all = p0.size
    out = {"unit": "params/s", "kind": "port", "nproc": cpus["nproc"], "affinity": cpus["affinity"],
           "cgroup_cpus": cpus["cgroup_cpus"], "threads": t16, "threads_all_cores": t_all}
    upd, reps, el = rate(n_all, g, 0.0, t16, seconds)
    out["update"] = upd
    out["value"] = upd
    out["cores"] = t16
    out["gbps"] = BYTES_UPDATE * upd / 1e9
    out["norm_clip_update"], reps_c, el_c = rate(n_all, g_clip, 1.0, t16, seconds)
    if t_all != t16:
        out["update_all_cores"], _, _ = rate(n_all, g, 0.0, t_all, seconds * 0.6)
        out["norm_clip_update_all_cores"], _, _ = rate(n_all, g_clip, 1.0, t_all, seconds * 0.6)
    else:
        out["update_all_cores"], out["norm_clip_update_all_cores"] = out["update"], out["norm_clip_update"]
    n1 = min(n_all, 4 * 1024 * 1024)                                 # one thread, first 4 Mi parameters
    out["single_thread"], _, _ = rate(n1, g, 0.0, 1, 2.0)
    out["single_thread_value"] = out["single_thread"]
    # the reference's own CPU-runnable case: one flat tensor of 1,048,576 parameters, full size (first Mi of the sample)
    n0 = 1 << 20
    r1, _, _ = rate(n0, g, 0.0, 1, 1.0)
    r16, _, _ = rate(n0, g, 0.0, t16, 1.0)
    out["flat_1m_ms_per_step_one_thread"] = n0 / r1 * 1e3
    out["flat_1m_ms_per_step_threads"] = n0 / r16 * 1e3
    out["sample"] = ("%d-param slice of embed_tokens (Qwen3-0.6B state after 99 steps), %d + %d passes of %.1f + %.1f s timed, "
                     "each from the saved state; update leg: g of step 100; norm+clip+update leg: g~N(0,5e-3), max_norm 1.0; "
                     "oracle's threaded AdamW loop, gcc -O3, no FMA contraction, static contiguous split over the threads"
                     % (n_all, reps, reps_c, el, el_c))
    return out


class HostList:
    """Host copies of the first `count` tensors of a ParamStore whose tensors are all FP16 (weights, gradients,
    moments as the pools hold them, padding between tensors included), for the CPU legs at full size; and a
    second copy of weights and moments, from which every timed pass starts."""

    def __init__(self, st, count):
        import numpy as np
        import torch
        assert all(s.dtype == 0 for s in st.specs[:count]), "HostList: FP16 tensors only"
        self.count = count
        self.sizes = [s.n for s in st.specs[:count]]
        self.off_pg, self.off = st.off_pg[:count], st.off[:count]
        end_pg, end = self.off_pg[-1] + self.sizes[-1], self.off[-1] + self.sizes[-1]
        half = lambda t, n: t[:n].view(torch.int16).cpu().numpy().view(np.uint16)
        self.p, self.g = half(st.p16, end_pg), half(st.g16, end_pg)
        self.m, self.v = st.m[:end].cpu().numpy(), st.v[:end].cpu().numpy()
        self.saved = (self.p.copy(), self.m.copy(), self.v.copy())
        self.params = sum(self.sizes)
        self.end_pg = end_pg

    def restore(self):
        self.p[:], self.m[:], self.v[:] = self.saved

    def gradients(self, st):
        """The store's present gradients of the same tensors (another leg's gradients)."""
        import numpy as np
        import torch
        return st.g16[:self.end_pg].view(torch.int16).cpu().numpy().view(np.uint16)


def cpu_list_legs(O, host, hl, hyper, step, threads, g_clip=None, per_tensor=False, budget=4.0, single_thread=True):
    """The oracle's threaded step over the whole tensor list held in `hl`, timed on the host: the update alone,
    optionally norm + clip + update with the gradients g_clip, optionally the update as one call per tensor, and
    the same legs on ONE thread.  Every timed pass starts from the saved state (restored outside the timed
    region; the port's speed depends on the values, see cpu_baseline).  Each leg: one untimed pass, then passes
    until `budget` seconds of wall time or 20 of them; a pass that takes more than half a second is timed once."""
    bc1, bc2 = host.bias_correction(hyper["beta1"], step), host.bias_correction(hyper["beta2"], step)
    args = (hyper["lr"], hyper["beta1"], hyper["beta2"], hyper["eps"], hyper["wd"], bc1, bc2)
    pools = (hl.off_pg, hl.off, hl.sizes)
    ptr_g = O.list_pointers(hl.p, hl.g, hl.m, hl.v, *pools)
    ptr_c = O.list_pointers(hl.p, g_clip, hl.m, hl.v, *pools) if g_clip is not None else None

    def timed(fn, warm=True):
        if warm:
            fn()
        reps, total, wall0 = 0, 0.0, time.perf_counter()
        while True:
            hl.restore()
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            total += dt
            reps += 1
            if dt > 0.5 or time.perf_counter() - wall0 >= budget or reps >= 20:
                return total / reps * 1e3, reps

    def update(th):
        return lambda: O.step_list_fp16_threaded(hl.p, hl.g, hl.m, hl.v, *pools, *args, 0.0, th, pointers=ptr_g)

    def clip(th):
        return lambda: O.step_list_fp16_threaded(hl.p, g_clip, hl.m, hl.v, *pools, *args, 1.0, th, pointers=ptr_c)

    out = {"params": hl.params, "tensors": hl.count, "threads": threads}
    ms, reps = timed(update(threads))
    out.update(update_ms=ms, update_params_per_s=hl.params / (ms * 1e-3), update_gbps=BYTES_UPDATE * hl.params / (ms * 1e-3) / 1e9,
               update_passes=reps)
    if g_clip is not None:
        ms, reps = timed(clip(threads))
        out.update(norm_clip_update_ms=ms, norm_clip_update_params_per_s=hl.params / (ms * 1e-3), norm_clip_update_passes=reps)
    if per_tensor:
        ms, reps = timed(lambda: O.update_per_tensor_fp16_threaded(hl.p, hl.g, hl.m, hl.v, *pools, *args, threads, pointers=ptr_g))
        out.update(per_tensor_loop_update_ms=ms, per_tensor_loop_passes=reps)
    if single_thread:
        big = hl.params > (1 << 26)              # a pass takes seconds: no warm-up pass
        ms, _ = timed(update(1), warm=not big)
        out.update(single_thread_update_ms=ms, single_thread_update_params_per_s=hl.params / (ms * 1e-3))
        if g_clip is not None:
            ms, _ = timed(clip(1), warm=not big)
            out.update(single_thread_norm_clip_update_ms=ms)
    hl.restore()
    return out


def graph_clip_step_ms(opt, B, warmup, steps):
    """norm + fused-clip update with device-resident hyper-parameters, recorded once as a HIP graph and replayed:
    what a caller of rlx_plan_adamw_scheduled pays per step when nothing comes from the host.  ms per replay."""
    import torch
    n = 2 * (warmup + steps) + 8
    opt.upload_schedule([opt.lr] * n)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = torch.cuda.current_stream().cuda_stream
            opt.plan.grad_norm(1.0, s)
            opt.step_scheduled(fused_clip=True, stream=s)
    torch.cuda.synchronize()
    ms = time_events(graph.replay, warmup, steps)
    opt.note_replayed_steps(warmup + steps)
    del graph
    return ms


def time_events(fn, warmup, steps):
    """ms per call: `steps` calls back to back between two events on torch's current stream (the stream
    every kernel here is launched on)."""
    import torch
    for _ in range(warmup):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def measure_workload(name, pkg, host, steps, warmup, chunk=0, O=None):
    """Update, norm and norm + fused-clip update of one of the secondary configurations, from seeded state.
    With the oracle `O` given, also the CPU legs of this configuration at its own size (under "cpu")."""
    import torch
    B, L = pkg.binding, pkg.layout
    master = False
    if name == "flat-1m":
        specs = [L.TensorSpec("flat", 1 << 20, L.DTYPE_F16, 0, 0)]
        p_std, g_std, what = 0.02, 1e-3, "one flat tensor of 1,048,576 FP16 parameters (22 MB: cache-resident)"
    elif name == "qwen3-0.6b-master":
        specs = L.qwen3_tensor_list(L.QWEN3_0_6B, norm_dtype=L.DTYPE_F32, reference_decay_groups=True)
        master, p_std, g_std = True, 0.02, 5e-3
        what = "Qwen3-0.6B in the reference's layout: FP32 norm weights, FP32 master copy, no decay on embedding and norms"
    elif name == "ragged":
        specs = L.ragged_tensor_list()
        p_std, g_std, what = 0.01, 1e-3, "4,096 tensors of 128..65,536 elements in one launch (cache-resident)"
    elif name == "qwen3-8b":
        specs = L.qwen3_tensor_list(L.QWEN3_8B)
        p_std, g_std, what = 0.02, 1e-4, "Qwen3-8B tensor list, untied lm_head, 98 GB resident, step 1000, clip active"
    else:
        raise SystemExit("unknown workload " + name)
    N = L.total_elements(specs)
    if N < (1 << 26):         # cache-resident: launches of a few microseconds need many repetitions to time
        steps, warmup = max(steps, 400), max(warmup, 50)
    st = host.ParamStore(specs, "cuda:0", master=master)
    st.fill("p", SEED_P, 1.0 if name == "ragged" else 0.0, p_std)
    st.fill("g", SEED_G, 0.0, g_std)
    st.fill("m", SEED_P + 1, 0.0, 1e-4)
    st.fill("v", SEED_P + 2, 1e-8, 1e-8, flags=B.FILL_ABS)
    if master:
        st.init_master()
    opt = host.AdamWOptimizer(st, lr=1e-5, chunk_elems=chunk)
    opt.step_ = 999
    stream = torch.cuda.current_stream().cuda_stream
    bpp = 28 if master else BYTES_UPDATE
    # the CPU legs first, on host copies of the seeded state as it is now: the timed GPU steps below repeat one step on
    # the same gradients and move the state on, and the CPU port's speed depends on the values
    cpu = None
    if O is not None and not master:
        hyper = dict(lr=1e-5, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)
        t16 = min(16, host_cpus()["affinity"])
        if name == "qwen3-8b":
            # a slice of at least 1e9 parameters: the leading tensors (embedding, lm_head ... in list order)
            count, tot = 0, 0
            while tot < 1_000_000_000:
                tot += specs[count].n
                count += 1
            hl = HostList(st, count)
            cpu = cpu_list_legs(O, host, hl, hyper, 1000, t16, g_clip=hl.g, budget=4.0, single_thread=False)
            cpu["sample"] = "the first %d tensors of the list (%d parameters); full-size figures extrapolated by parameter count" % (count, tot)
            for key in ("update_ms", "norm_clip_update_ms"):
                cpu["extrapolated_full_" + key] = cpu[key] * N / tot
        else:
            hl = HostList(st, len(specs))
            cpu = cpu_list_legs(O, host, hl, hyper, 1000, t16, g_clip=hl.g, per_tensor=(name == "ragged"), budget=2.0)
            cpu["sample"] = "the whole configuration"
        del hl
    upd = time_events(lambda: opt.step(), warmup, steps)
    nrm = time_events(lambda: opt.plan.grad_norm(1.0, stream), warmup, steps)

    def clip_step():
        opt.plan.grad_norm(1.0, stream)
        opt.step(fused_clip=True)

    both = time_events(clip_step, warmup, steps)
    norm, scale, _ = opt.plan.norm_read(stream)
    graph_ms = graph_clip_step_ms(opt, B, warmup, steps) if name != "qwen3-8b" else None
    scale_ms = time_events(lambda: opt.plan.scale_grads(stream), 1, 5)   # shrinks the gradients: last leg
    out = {
        "workload": what, "params": N, "tensors": len(specs), "bytes_per_param": bpp,
        "chunk_elems": opt.plan.chunk_elems, "chunks": opt.plan.num_chunks,
        "update_ms": upd, "update_gbps": bpp * N / (upd * 1e-3) / 1e9, "params_per_s": N / (upd * 1e-3),
        "norm_ms": nrm, "norm_gbps": BYTES_NORM * N / (nrm * 1e-3) / 1e9,
        "clip_step_ms": both, "clip_step_gbps": (bpp + BYTES_NORM) * N / (both * 1e-3) / 1e9,
        "grad_norm": norm, "clip_scale": scale, "scale_pass_ms": scale_ms, "unfused_clip_step_ms": both + scale_ms,
        "graph_clip_step_ms": graph_ms,
    }
    if cpu is not None:
        out["cpu"] = cpu
    out["update_frac_of_peak"] = out["update_gbps"] / HBM_PEAK_GBPS
    out["clip_step_frac_of_peak"] = out["clip_step_gbps"] / HBM_PEAK_GBPS
    if name == "ragged":      # against one flat tensor of the same element count
        del opt, st
        flat = host.ParamStore([L.TensorSpec("flat", N, L.DTYPE_F16, 0, 0)], "cuda:0")
        flat.fill("p", SEED_P, 1.0, p_std)
        flat.fill("g", SEED_G, 0.0, g_std)
        flat.fill("m", SEED_P + 1, 0.0, 1e-4)
        flat.fill("v", SEED_P + 2, 1e-8, 1e-8, flags=B.FILL_ABS)
        fopt = host.AdamWOptimizer(flat, lr=1e-5)
        fopt.step_ = 999
        if O is not None:      # the same element count as one flat tensor on the host
            hl = HostList(flat, 1)
            fcpu = cpu_list_legs(O, host, hl, dict(lr=1e-5, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01), 1000,
                                 min(16, host_cpus()["affinity"]), budget=2.0)
            out["cpu"]["flat_update_ms"] = fcpu["update_ms"]
            out["cpu"]["update_vs_flat"] = out["cpu"]["update_ms"] / fcpu["update_ms"]
            out["cpu"]["per_tensor_loop_vs_flat"] = out["cpu"]["per_tensor_loop_update_ms"] / fcpu["update_ms"]
            del hl
        out["flat_update_ms"] = time_events(lambda: fopt.step(), warmup, steps)
        out["flat_norm_ms"] = time_events(lambda: fopt.plan.grad_norm(1.0, stream), warmup, steps)

        def flat_clip_step():
            fopt.plan.grad_norm(1.0, stream)
            fopt.step(fused_clip=True)

        out["flat_clip_step_ms"] = time_events(flat_clip_step, warmup, steps)
        out["update_vs_flat"] = upd / out["flat_update_ms"]
        out["norm_vs_flat"] = nrm / out["flat_norm_ms"]
        out["clip_step_vs_flat"] = both / out["flat_clip_step_ms"]
        out["flat_graph_clip_step_ms"] = graph_clip_step_ms(fopt, B, warmup, steps)
        out["graph_clip_step_vs_flat"] = graph_ms / out["flat_graph_clip_step_ms"]
        del fopt, flat
    return out


def workload_line(name, w, steps, warmup, B):
    """The bench line of a secondary configuration (--workload)."""
    variant = B.get_tuning("update_variant")
    return {
        "metric": "AdamW params/sec, %s step" % name, "value": w["params_per_s"], "unit": "params/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": w["update_ms"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "storage": STORAGE, "data": "synthetic",
        "config": {"workload": w["workload"], "params": w["params"], "tensors": w["tensors"],
                   "bytes_per_param": w["bytes_per_param"], "chunk_elems": w["chunk_elems"], "chunks": w["chunks"],
                   "update_variant": variant},
        "roofline": {"bound": "hbm", "achieved": w["update_gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": w["update_gbps"] / HBM_PEAK_GBPS, "traffic": None, "traffic_source": None,
                     "kernel": B.update_variant_name(variant), "kernel_ms": w["update_ms"],
                     "algorithmic_bytes_per_launch": w["bytes_per_param"] * w["params"]},
        "cpu_baseline": w.get("cpu"),
        "measured": {k: v for k, v in w.items() if k not in ("workload", "params", "tensors", "cpu")},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="qwen3-0.6b",
                    help="qwen3-0.6b (default, the headline), flat-1m, qwen3-0.6b-master, ragged, qwen3-8b")
    ap.add_argument("--configs", default="all",
                    help="with the headline workload: 'all' (default) also measures the other configurations and "
                         "reports them under \"configs\"; 'none' skips them; or a comma-separated subset")
    ap.add_argument("--chunk", type=int, default=0, help="chunk_elems of the plan (0 = automatic)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--variant", type=int, default=None, help="update kernel form (tuning key update_variant)")
    ap.add_argument("--quick-setup", action="store_true",
                    help="seed the moments directly instead of running 99 steps (short profiler runs: few "
                         "dispatches); the parity sample then covers one step")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run the FP16->FP32 convert kernel on 2^28 elements (reads 512 MiB, writes 1 GiB): "
                         "a stream of known size against which profiler byte counters are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards by parameter "
            "range with one scalar all-reduce for the norm, which is not built)." % args.gpus)
        sys.exit(2)

    import numpy as np
    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    pkg = entry.load_package()
    host = importlib.import_module(entry.PKG_NAME + ".host")
    B, L = pkg.binding, pkg.layout
    B.load()
    O = entry.load_oracle()
    if args.variant is not None:
        B.set_tuning("update_variant", args.variant)
    if args.workload != "qwen3-0.6b":
        w = measure_workload(args.workload, pkg, host, args.steps, args.warmup, args.chunk, None if args.no_cpu else O)
        print(json.dumps(workload_line(args.workload, w, args.steps, args.warmup, B)), flush=True)
        return

    hyper = dict(lr=1e-5, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)
    specs = L.qwen3_tensor_list(L.QWEN3_0_6B)
    N = L.total_elements(specs)
    st = host.ParamStore(specs, "cuda:0")
    st.fill("p", SEED_P, 0.0, 0.02)
    opt = host.AdamWOptimizer(st, lr=hyper["lr"], beta1=hyper["beta1"], beta2=hyper["beta2"], eps=hyper["eps"],
                              weight_decay=hyper["wd"], chunk_elems=args.chunk)
    emb = [i for i, s in enumerate(specs) if s.name == "embed_tokens"][0]

    # ---- parity of a sample while the state is built: 99 seeded steps, oracle replays a slice ----
    samp = [(0, 0, 20000), (emb, 1024 * 5000, 30000), (len(specs) - 1, 0, 1024), (3, 2097152 - 4100, 4100)]

    def grab(which, i, lo, n):
        t = st.param(i) if which == "p" else st.grad(i) if which == "g" else st.state(i, which)
        t = t[lo: lo + n]
        return t.view(torch.int16).cpu().numpy().view(np.uint16).copy() if t.dtype == torch.float16 \
            else t.cpu().numpy().copy()

    torch.cuda.synchronize()
    first_step = 1
    if args.quick_setup:
        st.fill("m", SEED_P + 1, 0.0, 1e-5)
        st.fill("v", SEED_P + 2, 1e-9, 1e-9, flags=B.FILL_ABS)
        opt.step_ = 98
        first_step = 99
        torch.cuda.synchronize()
    ref = [dict(p=grab("p", i, lo, n), m=grab("m", i, lo, n), v=grab("v", i, lo, n)) for i, lo, n in samp]
    t_setup = time.perf_counter()
    for step in range(first_step, 100):
        st.fill("g", SEED_G + step, 0.0, 1e-4, zero_row_frac=0.9, only=("embed_tokens",))
        opt.step()
        for (i, lo, n), r in zip(samp, ref):
            g = O.fill_f16(n, L._hash64(SEED_G + step, i), 0.0, 1e-4, first=lo,
                           row_len=specs[i].row_len if i == emb else 0,
                           zero_rows_below=int(0.9 * 2 ** 32) if i == emb else 0)
            O.adamw_fp16(None, r["p"], g, r["m"], r["v"], hyper["lr"], hyper["beta1"], hyper["beta2"],
                         hyper["eps"], hyper["wd"], host.bias_correction(hyper["beta1"], step),
                         host.bias_correction(hyper["beta2"], step))
    torch.cuda.synchronize()
    for (i, lo, n), r in zip(samp, ref):
        for k in ("p", "m", "v"):
            got = grab(k, i, lo, n)
            assert np.array_equal(got, r[k]), "bench parity: tensor %d %s differs from the oracle" % (i, k)
    log("setup: %d seeded steps + sample parity ok (%.1f s)" % (100 - first_step, time.perf_counter() - t_setup))
    # gradients of the measured step (step 100)
    st.fill("g", SEED_G + 100, 0.0, 1e-4, zero_row_frac=0.9, only=("embed_tokens",))

    # ---- CPU baseline inputs: the state after exactly 99 steps and the gradients of step 100, taken BEFORE the timed
    # GPU steps (which repeat step 100 on the same gradients and so move the state on: the CPU port's speed depends on
    # the values, the GPU kernel's does not).  A slice of the embedding, and the whole configuration (7.2 GB). ----
    n_s = 32 * 1024 * 1024
    sample = None if args.no_cpu else tuple(grab(k, emb, 0, n_s) for k in ("p", "g", "m", "v"))
    host_list = None if args.no_cpu else HostList(st, len(specs))

    # ---- timed: update only (configs[1]) ----
    def run(fn, warmup, steps):
        """W untimed steps, then exactly `steps` launches back to back between two HIP events on the
        launch stream, bracketed by synchronisations.  Returns (wall seconds, event ms per step,
        per-step event ms from a second, separately instrumented pass)."""
        for _ in range(warmup):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ev_ms = a.elapsed_time(b) / steps
        k2 = min(steps, 20)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(k2 + 1)]
        ev[0].record()
        for k in range(k2):
            fn()
            ev[k + 1].record()
        torch.cuda.synchronize()
        return wall, ev_ms, [ev[k].elapsed_time(ev[k + 1]) for k in range(k2)]

    wall, ev_ms, per = run(lambda: opt.step(), args.warmup, args.steps)
    ms_per_step = wall * 1e3 / args.steps
    value = N * args.steps / wall
    kernel_ms = ev_ms
    achieved = BYTES_UPDATE * N / (kernel_ms * 1e-3) / 1e9


    # ---- timed: norm + clip scale + fused update (configs[2]); larger gradients so that clipping is active ----
    st.fill("g", SEED_G + 1000, 0.0, 5e-3)
    stream = torch.cuda.current_stream().cuda_stream
    g_clip = None if args.no_cpu else grab("g", emb, 0, n_s)
    g_clip_full = None if args.no_cpu else host_list.gradients(st)

    def clip_step():
        opt.plan.grad_norm(1.0, stream)
        opt.step(fused_clip=True)

    cwall, cev_ms, cper = run(clip_step, max(2, args.warmup // 2), max(5, args.steps // 2))
    norm, scale, _ = opt.plan.norm_read(stream)
    norm_ms = time_events(lambda: opt.plan.grad_norm(1.0, stream), 3, 20)
    clip = {"ms_per_step": cev_ms, "params_per_s": N / (cev_ms * 1e-3),
            "achieved_gbps": (BYTES_UPDATE + BYTES_NORM) * N / (cev_ms * 1e-3) / 1e9,
            "bytes_per_param": BYTES_UPDATE + BYTES_NORM, "grad_norm": norm, "clip_scale": scale,
            "norm_ms": norm_ms, "norm_gbps": BYTES_NORM * N / (norm_ms * 1e-3) / 1e9,
            "workload": "same list, g~N(0,5e-3), max_norm=1.0: norm pass + final pass + fused-clip update"}
    clip["frac_of_peak"] = clip["achieved_gbps"] / HBM_PEAK_GBPS
    # Where the clip step's time goes.  The plain and the fused-clip update are two kernels (the clip is a
    # compile-time choice): the plain one on this leg's dense gradients (the headline's have 23 % exact zeros from
    # the sparse embedding rows), and the fused-clip one alone, the scale already on the device.
    clip["dense_update_ms"] = time_events(lambda: opt.step(), 3, max(5, args.steps // 2))
    clip["fused_update_ms"] = time_events(lambda: opt.step(fused_clip=True), 3, max(5, args.steps // 2))
    clip["fused_update_gbps"] = BYTES_UPDATE * N / (clip["fused_update_ms"] * 1e-3) / 1e9
    clip["dense_update_gbps"] = BYTES_UPDATE * N / (clip["dense_update_ms"] * 1e-3) / 1e9
    clip["ms_minus_parts"] = cev_ms - clip["norm_ms"] - clip["fused_update_ms"]
    clip["graph_ms_per_step"] = graph_clip_step_ms(opt, B, 3, max(5, args.steps // 2))

    calibrate = None
    if args.calibrate:
        n_c = 1 << 28
        src = torch.zeros(n_c, dtype=torch.float16, device="cuda:0")
        dst = torch.empty(n_c, dtype=torch.float32, device="cuda:0")
        B.fill_f16(src.data_ptr(), n_c, 77, 0.0, 0.02, stream=stream)
        conv_ms = time_events(lambda: B.check(B.fp16_to_fp32(dst.data_ptr(), src.data_ptr(), n_c, stream),
                                              "rlx_fp16_to_fp32"), 2, 5)
        calibrate = {"kernel": "convert_tile_kernel", "elements": n_c, "bytes": 6 * n_c, "ms": conv_ms,
                     "gbps": 6 * n_c / (conv_ms * 1e-3) / 1e9}
        calibrate["frac_of_peak"] = calibrate["gbps"] / HBM_PEAK_GBPS
        del src, dst

    # ---- the separate scale pass of the unfused clip (4 bytes per FP16 gradient), last on this store: it
    # shrinks the gradients on every call; the scale stays the one that the clip leg left on the device ----
    scale_ms = time_events(lambda: opt.plan.scale_grads(stream), 1, 5)
    clip["scale_pass_ms"] = scale_ms
    clip["scale_pass_gbps"] = 4 * N / (scale_ms * 1e-3) / 1e9
    clip["unfused_ms_per_step"] = cev_ms + scale_ms
    chunk_elems, chunks = opt.plan.chunk_elems, opt.plan.num_chunks
    del opt, st
    torch.cuda.empty_cache()

    # ---- the other configurations, one after the other, each store freed before the next ----
    configs = {}
    wanted = [] if args.configs == "none" else list(SECONDARY) if args.configs == "all" else args.configs.split(",")
    for name in wanted:
        t0 = time.perf_counter()
        big = name == "qwen3-8b"
        configs[name] = measure_workload(name, pkg, host, 10 if big else min(args.steps, 50), 3 if big else min(args.warmup, 10),
                                         O=None if args.no_cpu else O)
        torch.cuda.empty_cache()
        log("config %s: update %.4f ms, norm %.4f ms, clip step %.4f ms (%.1f s)" % (
            name, configs[name]["update_ms"], configs[name]["norm_ms"], configs[name]["clip_step_ms"],
            time.perf_counter() - t0))

    # ---- CPU baseline on a bounded sample of the same workload ----
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(O, host, sample, g_clip, hyper, 100)
        # the configurations at their own sizes (the slice above stays for comparison with earlier runs)
        cpu["configs"] = {"qwen3-0.6b": cpu_list_legs(O, host, host_list, hyper, 100, cpu["threads"], g_clip=g_clip_full)}
        cpu["configs"]["qwen3-0.6b"]["sample"] = "the whole configuration: all 310 tensors, 7.2 GB of host state"
        for name, w in configs.items():
            if "cpu" in w:
                cpu["configs"][name] = w.pop("cpu")
        del host_list, g_clip_full

    # HBM bytes per launch of the update kernel as counted by the profiler: recorded beforehand with rocprofv3
    # (the counters cannot be read from inside this process), only valid for the shipped kernel and chunking
    traffic, traffic_source = None, None
    variant = B.get_tuning("update_variant")
    tpath = os.path.join(ROOT, "profiles", "adamw_tile_kernel_qwen3_0.6b_traffic.json")
    if variant == 0 and args.chunk == 0 and os.path.exists(tpath):
        try:
            traffic = json.load(open(tpath)).get("traffic_bytes_per_launch")
            traffic_source = "recorded, not measured in this run: profiles/adamw_tile_kernel_qwen3_0.6b_traffic.json " \
                             "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, scaled by a convert stream)"
        except Exception:
            traffic = None

    out = {
        "metric": "AdamW params/sec, Qwen3-0.6B step", "value": value, "unit": "params/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "storage": STORAGE,
        "data": "synthetic",
        "config": {"workload": "Qwen3-0.6B tensor list (310 tensors, 596,049,920 params), FP16 p/g, FP32 m/v, "
                               "step 100 after 99 seeded steps, g~N(0,1e-4) with 90% of embedding rows zero, "
                               "no clip; one multi-tensor launch per step",
                   "params": N, "tensors": len(specs), "bytes_per_param": BYTES_UPDATE,
                   "chunk_elems": chunk_elems, "chunks": chunks, "update_variant": variant},
        "hbm_gbps": BYTES_UPDATE * N * args.steps / wall / 1e9,
        "hbm_frac_of_peak": BYTES_UPDATE * N * args.steps / wall / 1e9 / HBM_PEAK_GBPS,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": B.update_variant_name(variant), "kernel_ms": kernel_ms,
                     "algorithmic_bytes_per_launch": BYTES_UPDATE * N,
                     "isolated_launch_ms_min": float(np.min(per)), "isolated_launch_ms_median": float(np.median(per))},
        "cpu_baseline": cpu,
        "clip_step": clip,
        "configs": configs,
        "parity": "4 sampled slices replayed by the CPU oracle over %d steps: bit-identical" % (100 - first_step),
    }
    # the figures of the other legs also as plain numbers inside "roofline", next to the headline kernel's
    # (records that keep only the standard objects of this line then still hold every configuration)
    flat = out["roofline"]
    flat["clip_step.ms"], flat["clip_step.gbps"] = clip["ms_per_step"], clip["achieved_gbps"]
    flat["clip_step.frac"], flat["clip_step.norm_ms"] = clip["frac_of_peak"], clip["norm_ms"]
    flat["clip_step.dense_update_ms"], flat["clip_step.fused_update_ms"] = clip["dense_update_ms"], clip["fused_update_ms"]
    flat["clip_step.graph_ms"] = clip["graph_ms_per_step"]
    for name, w in configs.items():
        for key in ("update_ms", "update_gbps", "norm_ms", "clip_step_ms", "clip_step_gbps", "flat_update_ms",
                    "flat_norm_ms", "flat_clip_step_ms", "graph_clip_step_ms", "flat_graph_clip_step_ms"):
            if w.get(key) is not None:
                flat["%s.%s" % (name, key)] = w[key]
    if calibrate:
        out["calibrate"] = calibrate
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
