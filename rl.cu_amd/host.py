"""Host side of the optimizer step on torch-allocated device memory.

Mirrors the reference's caller-facing interface for this path:
  AdamWOptimizer        include/training/optimizer.h:59-147  (public lr/beta1/beta2/eps/weight_decay,
                        set_lr, get_step, step)
  clip_grad_norm_       include/training/trainer.h:323-352    (returns the pre-clip norm)
  training_step order   include/training/trainer.h:279-286    (clip, then step)
torch is used for device memory and streams only; all arithmetic on tensors happens in
librlx_adamw.so.
"""
import ctypes as C
import json
import math
import os
import struct
import time

from . import binding as B
from .layout import DTYPE_F16, DTYPE_F32, _hash64

_libm = C.CDLL("libm.so.6")
_libm.powf.argtypes = [C.c_float, C.c_float]
_libm.powf.restype = C.c_float


def bias_correction(beta, step):
    """1 - powf(beta, (float)step), in FP32 as on the reference's host (optimizer.h:121-122)."""
    import numpy as np
    return float(np.float32(1.0) - np.float32(_libm.powf(beta, float(step))))


_libm.cosf.argtypes = [C.c_float]
_libm.cosf.restype = C.c_float


class LRScheduler:
    """Warm-up, then constant or cosine decay: the reference's LRScheduler
    (include/training/lr_scheduler.h:10-57) with the same methods, in FP32 step by step."""

    def __init__(self):
        self._cosine, self._base, self._min, self._warmup, self._total = False, 1e-5, 0.0, 0, 0

    def init_constant(self, base_lr, warmup_steps=0):
        self._cosine, self._base, self._min, self._warmup, self._total = False, base_lr, base_lr, warmup_steps, 0

    def init_cosine(self, base_lr, min_lr, warmup_steps, total_steps):
        self._cosine, self._base, self._min, self._warmup, self._total = True, base_lr, min_lr, warmup_steps, total_steps

    def get_lr(self, step):
        import numpy as np
        f = np.float32
        base, lo = f(self._base), f(self._min)
        if self._warmup > 0 and step < self._warmup:
            return float(base * (f(step + 1) / f(self._warmup)))
        decay = self._total - self._warmup
        if not self._cosine or decay <= 0:
            return float(base)
        prog = step - self._warmup
        if prog >= decay:
            return float(lo)
        phase = f(np.pi) * f(prog) / f(decay)
        cosine = f(0.5) * (f(1.0) + f(_libm.cosf(float(phase))))
        return float(lo + (base - lo) * cosine)


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


class ParamStore:
    """Flat device pools for a list of TensorSpec: FP16 and FP32 weights and gradients, FP32
    moments, optional FP32 master copy.  Every tensor starts on a 256-byte boundary."""

    ALIGN = 128  # elements

    def __init__(self, specs, device="cuda:0", master=False, zero_state=True):
        import torch
        self.specs = list(specs)
        self.device = torch.device(device)
        a = self.ALIGN
        self.off = []       # offset into m/v/master (all tensors, one index space)
        self.off_pg = []    # offset into the weight/gradient pool of the tensor's dtype
        tot, tot16, tot32 = 0, 0, 0
        for s in self.specs:
            self.off.append(tot)
            tot += (s.n + a - 1) // a * a
            if s.dtype == DTYPE_F16:
                self.off_pg.append(tot16)
                tot16 += (s.n + a - 1) // a * a
            else:
                self.off_pg.append(tot32)
                tot32 += (s.n + a - 1) // a * a
        self.total = sum(s.n for s in self.specs)
        mk = torch.zeros if zero_state else torch.empty
        self.p16 = torch.zeros(max(tot16, 1), dtype=torch.float16, device=self.device)
        self.g16 = torch.zeros(max(tot16, 1), dtype=torch.float16, device=self.device)
        self.p32 = torch.zeros(max(tot32, 1), dtype=torch.float32, device=self.device)
        self.g32 = torch.zeros(max(tot32, 1), dtype=torch.float32, device=self.device)
        self.m = mk(tot, dtype=torch.float32, device=self.device)
        self.v = mk(tot, dtype=torch.float32, device=self.device)
        self.master = mk(tot, dtype=torch.float32, device=self.device) if master else None

    # --- views ---------------------------------------------------------------------
    def _pg(self, i, which):
        s = self.specs[i]
        pool = {("p", DTYPE_F16): self.p16, ("g", DTYPE_F16): self.g16,
                ("p", DTYPE_F32): self.p32, ("g", DTYPE_F32): self.g32}[(which, s.dtype)]
        return pool[self.off_pg[i]: self.off_pg[i] + s.n]

    def param(self, i):
        return self._pg(i, "p")

    def grad(self, i):
        return self._pg(i, "g")

    def state(self, i, which):
        pool = {"m": self.m, "v": self.v, "master": self.master}[which]
        return pool[self.off[i]: self.off[i] + self.specs[i].n]

    def descs(self, extra_grad_only=()):
        """TensorDesc list in spec order; extra_grad_only: torch tensors that only take part in
        the norm and in the scale pass."""
        out = []
        for i, s in enumerate(self.specs):
            out.append(B.TensorDesc(
                self.param(i).data_ptr(), self.grad(i).data_ptr(),
                self.state(i, "m").data_ptr(), self.state(i, "v").data_ptr(),
                self.state(i, "master").data_ptr() if (self.master is not None and s.dtype == DTYPE_F16) else None,
                s.n, s.dtype, s.flags))
        import torch
        for t in extra_grad_only:
            dt = DTYPE_F16 if t.dtype == torch.float16 else DTYPE_F32
            out.append(B.TensorDesc(None, t.data_ptr(), None, None, None, t.numel(), dt, B.TENSOR_GRAD_ONLY))
        return out

    # --- seeded fills (on the device) --------------------------------------------------
    def fill(self, which, seed, mean, std, zero_row_frac=0.0, only=None, flags=0):
        """which: 'p', 'g', 'm', 'v'.  Tensor i uses seed hash(seed, i).  zero_row_frac applies to
        tensors named in `only` (default: none) and zeroes that share of their rows."""
        st = _stream()
        thresh = int(zero_row_frac * 2 ** 32) if zero_row_frac > 0 else 0
        for i, s in enumerate(self.specs):
            ts = _hash64(seed, i)
            masked = thresh and only is not None and s.name in only and s.row_len > 0
            row_len, zt = (s.row_len, thresh) if masked else (0, 0)
            if which in ("p", "g"):
                t = self._pg(i, which)
                fn = B.fill_f16 if s.dtype == DTYPE_F16 else B.fill_f32
            else:
                t = self.state(i, which)
                fn = B.fill_f32
            fn(t.data_ptr(), s.n, ts, mean, std, 0, flags, row_len, zt, st)

    def zero_grads(self, stream=None):
        """Clears both gradient pools (qwen3_gradients_zero, src/model/qwen3.cu:1109-1112)."""
        st = _stream() if stream is None else stream
        B.clear(self.g16.data_ptr(), self.g16.numel() * 2, st)
        B.clear(self.g32.data_ptr(), self.g32.numel() * 4, st)

    def init_master(self):
        """master = (float)param for FP16 tensors (optimizer.h:242)."""
        st = _stream()
        for i, s in enumerate(self.specs):
            if s.dtype == DTYPE_F16:
                B.check(B.fp16_to_fp32(self.state(i, "master").data_ptr(), self.param(i).data_ptr(), s.n, st),
                        "rlx_fp16_to_fp32")


class AdamWOptimizer:
    """Same public surface as the reference's AdamWOptimizer (optimizer.h:59-147), built from a
    ParamStore instead of a Qwen3Model*."""

    def __init__(self, store, lr=1e-4, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01,
                 chunk_elems=0, extra_grad_only=()):
        self.lr, self.beta1, self.beta2, self.eps, self.weight_decay = lr, beta1, beta2, eps, weight_decay
        self.store = store
        self.step_ = 0
        self._scheduled_lrs, self._scheduled_from = [], 0       # the uploaded step table and get_step() at its upload
        self.plan = B.Plan(store.descs(extra_grad_only), chunk_elems)

    def set_lr(self, new_lr):
        self.lr = new_lr

    def get_step(self):
        return self.step_

    def step_params(self):
        return B.StepParams(self.lr, self.beta1, self.beta2, self.eps, self.weight_decay,
                            bias_correction(self.beta1, self.step_), bias_correction(self.beta2, self.step_))

    def step(self, fused_clip=False, zero_grads=False, stream=None):
        """One launch over every tensor.  fused_clip: apply the scale that the last
        clip_grad_norm_(..., fused=True) left on the device.  zero_grads: clear every gradient
        buffer after it has been read (instead of qwen3_gradients_zero at the next step)."""
        self.step_ += 1
        flags = (B.CLIP_FUSED if fused_clip else 0) | (B.STEP_ZERO_GRADS if zero_grads else 0)
        self.plan.adamw(self.step_params(), flags, _stream() if stream is None else stream)

    # --- steps without the host (a recorded norm + update replayed step after step) ----------------------
    def upload_schedule(self, lrs, stream=None):
        """Uploads the hyper-parameters of the next len(lrs) steps (steps get_step()+1, ...): the given learning
        rates (from the LR scheduler) and the bias corrections 1 - powf(beta, t) computed here on the host, as
        optimizer.h:120-122 computes them.  Blocking; call outside the step loop."""
        steps = [B.StepParams(lr, self.beta1, self.beta2, self.eps, self.weight_decay,
                              bias_correction(self.beta1, self.step_ + 1 + k),
                              bias_correction(self.beta2, self.step_ + 1 + k)) for k, lr in enumerate(lrs)]
        self.plan.schedule_upload(steps, _stream() if stream is None else stream)
        self._scheduled_lrs = list(lrs)
        self._scheduled_from = self.step_

    def step_scheduled(self, fused_clip=False, zero_grads=False, stream=None):
        """step() with the hyper-parameters of the uploaded table; the device moves on to the next entry by
        itself, so a recorded launch can be replayed without any host write in between, through this window and
        every later upload (the recorded launch does not depend on the table's address or length).
        A call while torch's current stream is being captured records the launch and does not count as a step
        (count the replays with note_replayed_steps); an eager call counts, and raises if the table is used up
        or none was uploaded, instead of running with the last entry's learning rate and bias corrections."""
        import torch
        st = _stream() if stream is None else stream
        if not torch.cuda.is_current_stream_capturing():
            k = self.step_ - self._scheduled_from
            if not 0 <= k < len(self._scheduled_lrs):
                raise RuntimeError("step_scheduled: the uploaded table of %d steps is used up (or none was uploaded); "
                                   "call upload_schedule for the next window first" % len(self._scheduled_lrs))
            self.lr = self._scheduled_lrs[k]           # host-side bookkeeping only; the device reads its table
            self.step_ += 1
        flags = (B.CLIP_FUSED if fused_clip else 0) | (B.STEP_ZERO_GRADS if zero_grads else 0)
        self.plan.adamw_scheduled(flags, st)

    def note_replayed_steps(self, n):
        """After n replays of a recorded step_scheduled: get_step() += n.  Raises if that was more than the
        uploaded table held (the excess reused the table's last entry)."""
        self.step_ += n
        k = self.step_ - self._scheduled_from
        if 0 < k <= len(self._scheduled_lrs):
            self.lr = self._scheduled_lrs[k - 1]
        if k > len(self._scheduled_lrs):
            raise RuntimeError("%d scheduled steps have run since a table of %d was uploaded: the last %d reused the "
                               "table's last learning rate and bias corrections"
                               % (k, len(self._scheduled_lrs), k - len(self._scheduled_lrs)))

    # --- optimizer state on disk (the reference's save_checkpoint is a stub, trainer.h:317-319) ----
    # One format, shared with the C++ AdamWOptimizer (rl.cu_amd/host/training/optimizer.h): "RLXOPT02", int32
    # step, 5 x float32 (lr, beta1, beta2, eps, weight_decay), int32 sections; per section uint16 name length,
    # name, uint8 dtype (1 = FP32), int64 count, uint64 sum of the data's 32-bit words, data.  Sections, in this
    # order, each over a whole pool (all FP16 tensors in list order, then all FP32 tensors, without the padding
    # between tensors) and left out when empty: fp16.master (if kept), fp16.m, fp16.v, fp32.m, fp32.v.
    CKPT_MAGIC = b"RLXOPT02"
    CKPT_STAGE = 16 << 20            # elements per host staging buffer (64 MB)

    def _state_sections(self):
        """[(name, [tensor views in pool order], total count)] of this optimizer's state."""
        st = self.store
        idx16 = [i for i, s in enumerate(st.specs) if s.dtype == DTYPE_F16]
        idx32 = [i for i, s in enumerate(st.specs) if s.dtype == DTYPE_F32]
        out = []
        for pool, idx, kinds in (("fp16", idx16, (("master",) if st.master is not None else ()) + ("m", "v")),
                                 ("fp32", idx32, ("m", "v"))):
            for which in kinds:
                views = [st.state(i, which) for i in idx]
                total = sum(v.numel() for v in views)
                if total:
                    out.append((pool + "." + which, views, total))
        return out

    def _stage_chunks(self, views):
        for t in views:
            for lo in range(0, t.numel(), self.CKPT_STAGE):
                yield t[lo: lo + self.CKPT_STAGE]

    def save_state(self, path):
        """Writes step counter, hyper-parameters and the pooled m, v (and master) sections."""
        import numpy as np
        import torch
        torch.cuda.synchronize()
        secs = self._state_sections()
        tmp = path + ".tmp"
        with open(tmp, "wb") as f:
            f.write(self.CKPT_MAGIC)
            f.write(struct.pack("<i5fi", self.step_, self.lr, self.beta1, self.beta2, self.eps, self.weight_decay,
                                len(secs)))
            for name, views, total in secs:
                nb = name.encode()
                f.write(struct.pack("<H", len(nb)) + nb)
                f.write(struct.pack("<Bq", 1, total))
                sum_at = f.tell()
                f.write(struct.pack("<Q", 0))                  # patched once the data has passed
                csum = 0
                for part in self._stage_chunks(views):
                    a = part.detach().cpu().numpy()
                    csum = (csum + int(a.view(np.uint32).sum(dtype=np.uint64))) & 0xFFFFFFFFFFFFFFFF
                    f.write(a.tobytes())
                end = f.tell()
                f.seek(sum_at)
                f.write(struct.pack("<Q", csum))
                f.seek(end)
        os.replace(tmp, path)

    def load_state(self, path):
        """Restores what save_state (or the C++ class) wrote; the pools must have the same sizes.  The whole
        file is checked first; a foreign, truncated, damaged or differently laid out file raises ValueError (the
        message says which) and leaves the state untouched."""
        import numpy as np
        import torch
        secs = self._state_sections()
        data_at = []
        with open(path, "rb") as f:
            magic = f.read(8)
            if magic == b"RLXOPT01":
                raise ValueError("optimizer state in the older RLXOPT01 layout, which is no longer read: " + path)
            if magic != self.CKPT_MAGIC:
                raise ValueError("not an optimizer state file: " + path)
            head = f.read(28)
            if len(head) != 28:
                raise ValueError("truncated optimizer state file (header)")
            step, lr, b1, b2, eps, wd, nsec = struct.unpack("<i5fi", head)
            if step < 0 or not all(math.isfinite(x) for x in (lr, b1, b2, eps, wd)):
                raise ValueError("optimizer state with a negative step or a hyper-parameter that is not finite")
            if nsec != len(secs):
                raise ValueError("optimizer state has %d sections, this optimizer has %d (different layout: master "
                                 "copy or FP32 pool present on one side only)" % (nsec, len(secs)))
            for name, views, total in secs:                    # pass 1: headers and checksums, nothing is changed
                raw = f.read(2)
                if len(raw) != 2:
                    raise ValueError("truncated optimizer state file (section header)")
                (ln,) = struct.unpack("<H", raw)
                got = f.read(ln).decode(errors="replace")
                meta = f.read(17)
                if len(meta) != 17:
                    raise ValueError("truncated optimizer state file (section header)")
                dt, cnt, want = struct.unpack("<BqQ", meta)
                if got != name or dt != 1 or cnt != total:
                    raise ValueError("section %r with %d values where this optimizer needs %r with %d (different "
                                     "model or layout)" % (got, cnt, name, total))
                data_at.append(f.tell())
                csum, left = 0, total
                while left:
                    k = min(left, self.CKPT_STAGE)
                    a = np.fromfile(f, dtype=np.uint32, count=k)
                    if a.size != k:
                        raise ValueError("truncated optimizer state file (data of %s)" % name)
                    csum = (csum + int(a.sum(dtype=np.uint64))) & 0xFFFFFFFFFFFFFFFF
                    left -= k
                if csum != want:
                    raise ValueError("damaged optimizer state file: checksum mismatch in section " + name)
            if f.read(1):
                raise ValueError("optimizer state file is longer than its sections")
            for (name, views, total), at in zip(secs, data_at):     # pass 2: copy to the device
                f.seek(at)
                for part in self._stage_chunks(views):
                    a = np.fromfile(f, dtype=np.float32, count=part.numel())
                    part.copy_(torch.from_numpy(a))
        self.step_, self.lr, self.beta1, self.beta2, self.eps, self.weight_decay = step, lr, b1, b2, eps, wd
        torch.cuda.synchronize()

    def clip_grad_norm_(self, max_norm, fused=False, stream=None):
        """Returns the pre-clip norm (blocking read, as in the reference).  fused=False scales the
        gradients in place when norm > max_norm; fused=True leaves them alone and the following
        step(fused_clip=True) applies the scale."""
        st = _stream() if stream is None else stream
        self.plan.grad_norm(max_norm, st)
        norm, scale, _ = self.plan.norm_read(st)
        if not fused and norm > max_norm:
            self.plan.scale_grads(st)
        return norm


def training_step(optimizer, max_grad_norm, fused_clip=False, zero_grads=False):
    """The tail of Trainer::training_step (trainer.h:279-288): clip if max_grad_norm > 0, then step.
    Returns the pre-clip norm (0 if clipping is off)."""
    grad_norm = 0.0
    clipped = max_grad_norm > 0.0
    if clipped:
        grad_norm = optimizer.clip_grad_norm_(max_grad_norm, fused=fused_clip)
    optimizer.step(fused_clip=fused_clip and clipped, zero_grads=zero_grads)
    return grad_norm


def accumulation_step(optimizer, micro_batch, grad_accum_steps, max_grad_norm, loss_grad=None, fused_clip=False,
                      freeze=None, stream=None):
    """Trainer::training_step around the optimizer (include/training/trainer.h:231-289): clear the gradient
    pools; for each of grad_accum_steps micro-batches call micro_batch(k, scale_loss_grad) -> loss, which
    stands for forward, compute_loss and backward: it fills `loss_grad` (a torch FP32 tensor), calls
    scale_loss_grad() where the reference launches scale_grad_kernel (between compute_loss and backward,
    trainer.h:261-263) and adds its gradients into the pools; then clear the gradients of the tensor views
    in `freeze` (freeze_embed), clip, step.  Returns (mean loss, pre-clip norm)."""
    import numpy as np
    st = _stream() if stream is None else stream
    optimizer.store.zero_grads(st)
    scale = float(np.float32(1.0) / np.float32(grad_accum_steps))

    def scale_loss_grad():
        if loss_grad is not None:
            B.scale_f32(loss_grad.data_ptr(), scale, loss_grad.numel(), st)

    accum = 0.0
    for k in range(grad_accum_steps):
        accum += micro_batch(k, scale_loss_grad)
    for t in (freeze or ()):
        B.clear(t.data_ptr(), t.numel() * t.element_size(), st)
    grad_norm = training_step(optimizer, max_grad_norm, fused_clip=fused_clip)
    return accum / grad_accum_steps, grad_norm


class Logger:
    """JSON-lines metrics logger with the reference's interface (include/training/logger.h:27-128):
    log() accumulates, commit() writes the window's means as one object with a "step" key, appends to
    <log_dir>/train_log.jsonl and prints a summary line.  Keys come out sorted, as the reference's
    JSON object type orders them."""

    def __init__(self, log_dir=""):
        self._file, self._path, self._pending, self._history = None, "", {}, []
        if log_dir:
            self.open(log_dir)

    def open(self, log_dir):
        if not log_dir:
            return
        os.makedirs(log_dir, exist_ok=True)
        self._path = os.path.join(log_dir, "train_log.jsonl")
        self._file = open(self._path, "a")          # append: survives restarts

    def log(self, step, key, value=None):
        if isinstance(key, dict):
            for k, v in key.items():
                self.log(step, k, v)
            return
        import numpy as np
        acc = self._pending.setdefault(key, [np.float32(0.0), 0])
        acc[0] = np.float32(acc[0] + np.float32(value))       # FP32 accumulation, as the reference's
        acc[1] += 1

    def commit(self, step):
        if not self._pending:
            return
        import numpy as np
        obj = {"step": step}
        parts = ["[step %d]" % step]
        for key in sorted(self._pending):
            total, count = self._pending[key]
            val = float(total / np.float32(count)) if count else 0.0
            obj[key] = val
            parts.append(("  %s=%.3e" if (abs(val) < 0.01 and val != 0.0) else "  %s=%.4f") % (key, val))
        print("".join(parts))
        if self._file:
            self._file.write(json.dumps(obj, sort_keys=True, separators=(",", ":")) + "\n")
            self._file.flush()
        self._history.append(obj)
        self._pending = {}

    def history(self):
        return self._history

    def last(self, key):
        for obj in reversed(self._history):
            if key in obj:
                return obj[key]
        return math.nan

    def log_path(self):
        return self._path

    def close(self):
        if self._file:
            self._file.close()
            self._file = None


def train_loop(optimizer, scheduler, logger, produce_grads, total_steps, max_grad_norm=1.0, fused_clip=True,
               logging_steps=1, save_steps=0, save_path=None, tokens_per_step=0):
    """The optimizer end of Trainer::train (include/training/trainer.h:183-225): per step set the
    scheduled rate, obtain gradients (produce_grads(step) stands for forward/backward and returns the
    loss), clip, step, synchronise, log loss / lr / grad_norm / step_ms / tok_per_sec, commit every
    logging_steps, save the optimizer state every save_steps."""
    import torch
    global_step = 0
    while global_step < total_steps:
        cur_lr = scheduler.get_lr(global_step)
        optimizer.set_lr(cur_lr)
        t0 = time.perf_counter()
        loss = produce_grads(global_step)
        grad_norm = training_step(optimizer, max_grad_norm, fused_clip=fused_clip)
        torch.cuda.synchronize()
        step_ms = (time.perf_counter() - t0) * 1e3
        global_step += 1
        logger.log(global_step, "loss", loss)
        logger.log(global_step, "lr", cur_lr)
        logger.log(global_step, "grad_norm", grad_norm)
        logger.log(global_step, "step_ms", step_ms)
        logger.log(global_step, "tok_per_sec", tokens_per_step / (step_ms * 1e-3) if step_ms > 0 else 0.0)
        if global_step % logging_steps == 0:
            logger.commit(global_step)
        if save_steps > 0 and save_path and global_step % save_steps == 0:
            optimizer.save_state(save_path)
    return global_step
