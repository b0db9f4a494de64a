"""The elementwise end of an optimizer step (grafting + AdamW / SGD update) for all parameters of
a group in two launches of libqtensor_hip.so instead of a dozen torch kernels per parameter.

Arithmetic of the reference's step(): optimizers/shampoo1.py:310-331 (SGD), :405-427 (AdamW)
and the same lines of shampoo2.py.
"""
import ctypes as ct
import math

import torch

import qtensor.functional as F

if F.lib is not None:
    F.lib.qtensor_hip_tail_chunk.restype = ct.c_int
    F.lib.qtensor_hip_tail_chunk.argtypes = []
    F.lib.qtensor_hip_adamw_tail.restype = None
    F.lib.qtensor_hip_adamw_tail.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_void_p, ct.c_int, ct.c_double, ct.c_double,
                                             ct.c_double, ct.c_double, ct.c_double, ct.c_longlong, ct.c_void_p]
    F.lib.qtensor_hip_adamw_tail_rows.restype = None
    F.lib.qtensor_hip_adamw_tail_rows.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_void_p, ct.c_int, ct.c_double, ct.c_double,
                                                  ct.c_double, ct.c_double, ct.c_double, ct.c_void_p, ct.c_void_p]
    F.lib.qtensor_hip_sgd_tail.restype = None
    F.lib.qtensor_hip_sgd_tail.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_void_p, ct.c_int, ct.c_double, ct.c_double,
                                           ct.c_double, ct.c_int, ct.c_void_p]


class TailPlan:
    """Device-side table of (param, direction, grad, moment buffers) rows and the chunk map the
    kernels walk.  Rebuilt only when a buffer has moved."""

    def __init__(self):
        if F.lib is None:
            raise RuntimeError("libqtensor_hip.so is not available")
        self.chunk = F.lib.qtensor_hip_tail_chunk()
        self.key = None
        self.keep = None
        self.partial = None

    def _prepare(self, params, dirs, grads, m, v, graft):
        # (the gradient's address only where the row is grafted: the kernels do not read it otherwise)
        key = tuple((p.data_ptr(), d.data_ptr(), g.data_ptr() if f else 0, a.data_ptr(), 0 if b is None else b.data_ptr(), bool(f))
                    for p, d, g, a, b, f in zip(params, dirs, grads, m, v, graft))
        if key == self.key:
            return
        rows, owner, first = [], [], 0
        for i, (p, d, g, a, b, f) in enumerate(zip(params, dirs, grads, m, v, graft)):
            tensors = [p, d, a] + ([g] if f else []) + ([] if b is None else [b])
            for t in tensors:
                if not t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != p.numel():
                    raise ValueError("the fused update takes contiguous fp32 GPU tensors of equal size per parameter")
            chunks = -(-p.numel() // self.chunk)
            rows.append([p.data_ptr(), d.data_ptr(), g.data_ptr() if f else 0, a.data_ptr(), 0 if b is None else b.data_ptr(),
                         p.numel(), first, 1 if f else 0])
            owner += [i] * chunks
            first += chunks
        dev = params[0].device
        # through pinned memory and without blocking: a pageable copy would make the host wait for
        # everything the step has queued so far
        self.table = torch.tensor(rows, dtype=torch.int64).pin_memory().to(dev, non_blocking=True)
        self.owner = torch.tensor(owner, dtype=torch.int32).pin_memory().to(dev, non_blocking=True)
        if self.partial is None or self.partial.numel() != 2 * max(first, 1) or self.partial.device != dev:
            self.partial = torch.empty(2 * max(first, 1), dtype=torch.float32, device=dev)
        self.n_chunks = first
        self.any_graft = any(graft)
        self.key = key
        # The table holds raw addresses.  Parameters and moment buffers are kept alive here; gradients and directions
        # are not: they are only read by the launch that follows, while their owners still hold them, and keeping
        # them would pin one full set of gradients after zero_grad(set_to_none=True).  A tensor that comes back at
        # another address changes the key and the table is rebuilt.
        self.keep = (list(params), list(m), list(v))

    def adamw(self, params, dirs, grads, exp_avg, exp_avg_sq, graft, lr, betas, eps, weight_decay, step):
        """step: one count for all parameters, or a list with one count per parameter (the reference counts per
        parameter: optimizers/shampoo2.py:335-342); counts that differ go up as per-row bias corrections."""
        self._prepare(params, dirs, grads, exp_avg, exp_avg_sq, graft)
        steps = [step] * len(params) if isinstance(step, int) else list(step)
        if all(s == steps[0] for s in steps):
            F._call(F.lib.qtensor_hip_adamw_tail, params[0].device, self.table.data_ptr(), self.owner.data_ptr(), self.n_chunks,
                    self.partial.data_ptr(), int(self.any_graft), lr, betas[0], betas[1], eps, weight_decay, steps[0])
            return
        rows = [[math.sqrt(1.0 - betas[1] ** s), -lr / (1.0 - betas[0] ** s)] for s in steps]
        corrections = torch.tensor(rows, dtype=torch.float32).pin_memory().to(params[0].device, non_blocking=True)
        F._call(F.lib.qtensor_hip_adamw_tail_rows, params[0].device, self.table.data_ptr(), self.owner.data_ptr(), self.n_chunks,
                self.partial.data_ptr(), int(self.any_graft), lr, betas[0], betas[1], eps, weight_decay, corrections.data_ptr())
        self.corrections = corrections          # kept until the next call: the launch reads it asynchronously

    def sgd(self, params, dirs, grads, momentum_bufs, graft, lr, momentum, weight_decay, nesterov):
        self._prepare(params, dirs, grads, momentum_bufs, [None] * len(params), graft)
        F._call(F.lib.qtensor_hip_sgd_tail, params[0].device, self.table.data_ptr(), self.owner.data_ptr(), self.n_chunks,
                self.partial.data_ptr(), int(self.any_graft), lr, momentum, weight_decay, int(bool(nesterov)))
