"""TEST INFRASTRUCTURE, NOT PRODUCT CODE -- CPU restatement of the reference's "naive" low-bit
Shampoo preconditioner with the bit width FORCED to 4/8 on the CPU.

The reference never quantizes on the CPU (optimizers/shampoo1.py:125-128 sets the bit width to
32 there), so its own optimizer cannot serve as the low-bit CPU baseline.  This file strings the
reference's steps together the way its GPU path would run them, on top of the quantizer oracle:

  optimizers/shampoo1.py:35-99     block partitioning            -> pieces / blocks
  optimizers/shampoo1.py:148-179   statistics update             -> RefPreconditioner.add_statistics
  optimizers/shampoo1.py:181-201   inverse 4th roots (Newton)    -> .compute_preconditioners
  optimizers/shampoo1.py:203-241   preconditioned gradient       -> .preconditioned_grad
  optimizers/matrix_functions.py:21-141  power iteration, coupled Newton -> power_iteration / newton_root
  qtensor/functional.py:239-368 via oracle/quant_np.py (C form, or the per-segment torch loop
  when `loop=True`, which is what the reference's CPU code path would execute and what bench.py
  times as the CPU baseline).

Pins: the dense (32-bit) behaviour of the same steps is pinned by the reference runs stored in
tests/golden/reference_vectors.npz through tests/test_shampoo_oracle.py (this file run with
bits=32 must reproduce them); the quantizer underneath is pinned in tests/test_oracle_quant.py.
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.
"""
from __future__ import annotations

import numpy as np
import torch

from oracle import quant_loop_torch as QL
from oracle import quant_np as Q


def pieces(extent: int, block: int):
    if block > 0 and extent > block:
        cuts = (extent - 1) // block
        return [block] * cuts + [extent - cuts * block]
    return [extent]


def power_iteration(mat, v0, tol=1e-6, iters=10):
    v, value, change, used = v0.to(mat.dtype).clone(), 0.0, 1.0, 0
    while change > tol and used < iters:
        v = v / torch.norm(v)
        w = torch.mv(mat, v)
        s = torch.dot(v, w)
        change = torch.abs(s - value)
        v, value = w, s
        used += 1
    return value


def newton_root(mat, p, eps, v0, iters=10, tol=1e-6):
    """(mat + eps*lambda_max*I)^(-1/p); mat is modified like in the reference."""
    n = mat.shape[0]
    eye = torch.eye(n, dtype=mat.dtype)          # (float64 input: the same iteration in double, used as a yardstick)
    if n == 1:
        return eye
    w = -1.0 / p
    mat += (eps * power_iteration(mat, v0)) * eye
    z = (1 + p) / (2 * torch.norm(mat))
    root = eye * torch.pow(z, 1.0 / p)
    m = mat * z
    err = torch.max(torch.abs(m - eye))
    count = 0
    while err > tol and count < iters:
        t = (1 - w) * eye + w * m
        cand = root @ t
        tp, done = t, 1
        while done < p:
            tp = tp @ tp
            done *= 2
        m = tp @ m
        new_err = torch.max(torch.abs(m - eye))
        if new_err > err * 1.2:
            break
        root, err = cand, new_err
        count += 1
    return root


class _Slot:
    """One square matrix stored dense (bits 32) or as 4/8-bit codes with an exact diagonal."""

    def __init__(self, mat, bits, code, blocksize, min_lowbit_size, loop):
        self.order = mat.shape[0]
        self.low = bits in (4, 8) and mat.numel() >= min_lowbit_size
        self.bits, self.code, self.bs, self.loop = bits, code, blocksize, loop
        self.put(mat)

    def put(self, mat):
        if not self.low:
            self.dense = mat.clone()
        elif self.loop:
            self.q = QL.quantize_loop(mat.contiguous(), torch.from_numpy(self.code), self.order, self.bs, self.bits, True)
        else:
            self.q = Q.quantize_c(mat.numpy(), self.code, self.order, self.bs, self.bits, True)

    def get(self):
        if not self.low:
            return self.dense.clone()
        if self.loop:
            out, absmax, diag = self.q
            return QL.dequantize_loop(out, torch.from_numpy(self.code), self.order, absmax, self.bs, self.bits, diag=diag)
        out, absmax, diag = self.q
        return torch.from_numpy(Q.dequantize_c(out, self.code, self.order, absmax, self.bs, self.bits, diag=diag).copy())

    def codes(self):
        out, absmax, diag = self.q
        return (np.asarray(out), np.asarray(absmax), np.asarray(diag))


class RefPreconditioner:
    def __init__(self, shape, code, stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1200, prec_bits=4,
                 min_lowbit_size=4096, quan_blocksize=64, loop=False, root_dtype=torch.float32):
        # root_dtype=torch.float64 runs the Newton iteration in double on the same stored statistics: not the
        # reference's arithmetic, but the yardstick for how far fp32 rounding alone moves an inverse root
        dims = [d for d in shape if d != 1]
        self.shape = tuple(shape)
        self.rank2 = len(dims) > 1
        self.root_dtype = root_dtype
        self.beta, self.eps = stat_decay, matrix_eps
        self.active = False
        self.stats, self.precs = [], []
        if not self.rank2:
            return
        self.m, self.n = dims[0], int(np.prod(dims)) // dims[0]
        self.rows, self.cols = pieces(self.m, prec_maxorder), pieces(self.n, prec_maxorder)
        args = (prec_bits, code, quan_blocksize, min_lowbit_size, loop)
        for bm in self.rows:
            for bn in self.cols:
                for order in (bm, bn):
                    self.stats.append(_Slot(matrix_eps * torch.eye(order), *args))
                    self.precs.append(_Slot(torch.eye(order), *args))

    def blocks(self, grad):
        g = grad.reshape(self.m, self.n)
        out, r0 = [], 0
        for bm in self.rows:
            c0 = 0
            for bn in self.cols:
                out.append(g[r0:r0 + bm, c0:c0 + bn])
                c0 += bn
            r0 += bm
        return out

    def add_statistics(self, grad):
        if not self.rank2:
            return
        w1 = self.beta
        w2 = 1.0 if w1 == 1.0 else 1.0 - w1
        for j, blk in enumerate(self.blocks(grad)):
            blk = blk.float()
            for side in (0, 1):
                gram = blk @ blk.T if side == 0 else blk.T @ blk
                slot = self.stats[2 * j + side]
                cur = slot.get()
                cur.mul_(w1).add_(gram, alpha=w2)
                slot.put(cur)

    def compute_preconditioners(self, v0s):
        """v0s: one start vector per statistic, in storage order."""
        for slot, prec, v0 in zip(self.stats, self.precs, v0s):
            stat = slot.get().to(self.root_dtype)
            root = newton_root(stat, 4, self.eps, v0).float()
            if not slot.low:
                slot.dense = stat.float()  # the reference's in-place ridge on a dense statistic
            prec.put(root)
        self.active = True

    def preconditioned_grad(self, grad):
        if not self.rank2:
            return grad
        outs = []
        for j, blk in enumerate(self.blocks(grad)):
            outs.append(self.precs[2 * j].get() @ blk @ self.precs[2 * j + 1].get())
        rows, k = [], 0
        for _ in self.rows:
            rows.append(torch.cat(outs[k:k + len(self.cols)], dim=1))
            k += len(self.cols)
        return torch.cat(rows, dim=0).reshape(self.shape)
