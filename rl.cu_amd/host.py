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

from . import binding as B
from .layout import DTYPE_F16, DTYPE_F32, _hash64

_libm = C.CDLL("libm.so.6")
_libm.powf.argtypes = [C.c_float, C.c_float]
_libm.powf.restype = C.c_float


def bias_correction(beta, step):
    """1 - powf(beta, (float)step), in FP32 as on the reference's host (optimizer.h:121-122)."""
    import numpy as np
    return float(np.float32(1.0) - np.float32(_libm.powf(beta, float(step))))


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
