"""TEST INFRASTRUCTURE, NOT PRODUCT CODE -- CPU restatement of the reference's eigenbasis
("ours") low-bit Shampoo preconditioner with the bit width FORCED to 4/8 on the CPU.

The reference never quantizes on the CPU (optimizers/shampoo2.py:134 sets the bit width to 32
there), so its own optimizer cannot serve as the low-bit CPU checker.  This file strings the
reference's steps together the way its GPU path would run them, on top of the quantizer oracle:

  qtensor/utils.py:126-153         start: identity basis, quotients eps     -> RefEigenSlot.__init__
  qtensor/utils.py:156-171         QR(L Vt^T), Rayleigh quotients, keep the smaller half,
                                   store V^T through the plain quantizer    -> RefEigenSlot.quantize
  qtensor/utils.py:192-203         dequantize, rect_t1 Bjorck steps,
                                   V_keep^T diag(S) V_keep                  -> RefEigenSlot.dequantize
  qtensor/utils.py:205-227 and
  qtensor/functional.py:749-762    inverse root from the kept eigenpairs    -> RefEigenSlot.computepower
  optimizers/shampoo2.py:169-200   statistics update                        -> RefPreconditioner2.add_statistics
  optimizers/shampoo2.py:202-232   inverse 4th roots, mode 0 and 1          -> .compute_preconditioners
  optimizers/shampoo2.py:234-272   preconditioned gradient                  -> .preconditioned_grad
  (power iteration, coupled Newton and the exact-diagonal slots of the preconditioners come from
  oracle/shampoo_ref.py; the quantizer from oracle/quant_np.py, or the per-segment torch loop
  with `loop=True`, which is what the reference's CPU code path would execute and what bench.py
  times as the CPU baseline.)

Column signs.  The Q factor of a QR factorisation is unique only up to the signs of its columns;
the reference takes whatever LAPACK returns (utils.py:157).  Everything derived from the basis
(rebuilt statistic, quotients, inverse roots) does not depend on them, the stored 4-bit codes do
(the code table is not symmetric around zero).  With `positive_r=True` the columns are flipped so
that R has a positive diagonal -- the one choice every QR algorithm can reproduce -- and only then
are stored codes comparable with another implementation.

Pins: run dense (bits=32) this file must reproduce the reference's own shampoo2 runs stored in
tests/golden/reference_vectors.npz (pre_s2m0_*, pre_s2m1_*, svd_*, cp_*) through
tests/test_shampoo2_oracle.py; the low-bit flow is that same flow with the pinned quantizer in
between (checked there by hand for one update).
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.
"""
from __future__ import annotations

import numpy as np
import torch

from oracle import quant_loop_torch as QL
from oracle import quant_np as Q
from oracle.shampoo_ref import _Slot, newton_root, pieces


def bjorck(rows, steps):
    """`steps` times V <- 1.5 V - 0.5 V V^T V (utils.py:195-196, functional.py:756-757)."""
    for _ in range(steps):
        rows = 1.5 * rows - 0.5 * rows @ rows.T @ rows
    return rows


def orthonormal_factor(mat, positive_r=False):
    """Q of a Householder QR of mat (utils.py:157); optionally with the signs that make diag(R) > 0."""
    q, r = torch.linalg.qr(mat)
    if positive_r:
        s = torch.sign(torch.diagonal(r))
        s[s == 0] = 1.0
        q = q * s.unsqueeze(0)
    return q


class RefEigenSlot:
    """One PSD statistic L ~ Vt[keep]^T diag(S) Vt[keep] with Vt dense (bits 32) or held as plain
    4/8-bit codes (no exact diagonal)."""

    def __init__(self, order, eps, bits, code, blocksize, min_lowbit_size, rect_t1=1, rect_t2=4, loop=False,
                 positive_r=False):
        self.order, self.rect_t1, self.rect_t2 = order, rect_t1, rect_t2
        self.read_dtype = torch.float32      # float64: Bjorck steps and rebuilt statistic in double (a yardstick, see below)
        self.low = bits in (4, 8) and order * order >= min_lowbit_size
        self.bits, self.code, self.bs, self.loop, self.positive_r = bits, code, blocksize, loop, positive_r
        keep = max(1, order // 2)
        self.keep = torch.arange(order, dtype=torch.int64)[:keep]
        # var[0][0] * diag(I): every start quotient is eps, the largest one too (utils.py:137-141)
        self.svalue = torch.full((keep,), eps, dtype=torch.float32)
        self.max_eig = torch.tensor(eps, dtype=torch.float32)
        self._store(torch.eye(order))

    # ---- the basis, through the plain quantizer --------------------------------------------------
    def _store(self, vt):
        if not self.low:
            self.dense = vt.clone()
        elif self.loop:
            self.q = QL.quantize_loop(vt.contiguous(), torch.from_numpy(self.code), self.order, self.bs, self.bits, False)[:2]
        else:
            self.q = Q.quantize_c(vt.contiguous().numpy(), self.code, self.order, self.bs, self.bits, False)[:2]

    def basis(self):
        """The stored Vt as it comes back from the dequantizer (no Bjorck step)."""
        if not self.low:
            return self.dense
        out, absmax = self.q
        if self.loop:
            return QL.dequantize_loop(out, torch.from_numpy(self.code), self.order, absmax, self.bs, self.bits)
        return torch.from_numpy(Q.dequantize_c(out, self.code, self.order, absmax, self.bs, self.bits).copy())

    def codes(self):
        out, absmax = self.q
        return np.asarray(out), np.asarray(absmax)

    def load(self, codes, absmax, svalue, keep, max_eig):
        """Adopt a stored state (used to start two implementations from identical bits)."""
        self.q = (np.ascontiguousarray(codes, dtype=np.uint8), np.ascontiguousarray(absmax, dtype=np.float32))
        if self.loop:
            self.q = tuple(torch.from_numpy(x) for x in self.q)
        self.svalue = torch.as_tensor(svalue, dtype=torch.float32).clone()
        self.keep = torch.as_tensor(keep, dtype=torch.int64).clone()
        self.max_eig = torch.as_tensor(max_eig, dtype=torch.float32).clone()

    # ---- utils.py:192-203 ----------------------------------------------------------------------
    def dequantize(self):
        vt = bjorck(self.basis().to(self.read_dtype), self.rect_t1) if self.low else self.dense
        rows = vt[self.keep]
        return rows.T @ self.svalue.to(vt.dtype).diag() @ rows, vt

    # ---- utils.py:156-171 ----------------------------------------------------------------------
    def quantize(self, stat, vt):
        stat = stat.float()
        v = orthonormal_factor(stat @ vt.T.float(), self.positive_r)
        quotients = (v.T @ stat @ v).diag()
        keep = max(1, quotients.numel() // 2)
        ascending, where = torch.sort(quotients)
        self.keep = where[:keep].to(torch.int64)
        self.svalue = ascending[:keep].clone()
        self.max_eig = quotients.max().clone()
        self.quotients = quotients           # (kept for tests: how well separated the cut is)
        self._store(v.T.contiguous())

    # ---- utils.py:205-227 with functional.py:749-762 ------------------------------------------
    def computepower(self, p, ridge_epsilon, steps=None):
        if steps is None:
            steps = self.rect_t2 if self.low else 0
        rows = bjorck(self.basis()[self.keep].to(self.read_dtype), steps)
        rho = ridge_epsilon * self.max_eig
        weights = (1 / (self.svalue + rho).pow(1 / p)).to(rows.dtype)
        return rows.T @ weights.diag() @ rows


class RefPreconditioner2:
    def __init__(self, shape, code, stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1200, prec_bits=4,
                 min_lowbit_size=4096, quan_blocksize=64, rect_t1=1, rect_t2=4, inv_root_mode=0, loop=False,
                 positive_r=False):
        # (root_dtype, set by tests to torch.float64 before compute_preconditioners: the inverse roots -- Bjorck
        # steps, rebuilt statistic, Newton iteration -- in double on the same stored state; not the reference's
        # arithmetic, but the yardstick for how far fp32 rounding alone moves an inverse root)
        self.root_dtype = torch.float32
        dims = [d for d in shape if d != 1]
        self.shape = tuple(shape)
        self.rank2 = len(dims) > 1
        self.beta, self.eps, self.mode = stat_decay, matrix_eps, inv_root_mode
        self.active = False
        self.stats, self.precs = [], []
        if not self.rank2:
            return
        self.m, self.n = dims[0], int(np.prod(dims)) // dims[0]
        self.rows, self.cols = pieces(self.m, prec_maxorder), pieces(self.n, prec_maxorder)
        for bm in self.rows:
            for bn in self.cols:
                for order in (bm, bn):
                    self.stats.append(RefEigenSlot(order, matrix_eps, prec_bits, code, quan_blocksize, min_lowbit_size,
                                                   rect_t1, rect_t2, loop, positive_r))
                    self.precs.append(_Slot(torch.eye(order), prec_bits, code, quan_blocksize, min_lowbit_size, loop))

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
                cur, vt = slot.dequantize()
                cur = cur.clone()
                cur.mul_(w1).add_(gram, alpha=w2)
                slot.quantize(cur, vt)

    def compute_preconditioners(self, v0s=None):
        """v0s (mode 1 only): one power-iteration start vector per statistic, in storage order."""
        for i, (slot, prec) in enumerate(zip(self.stats, self.precs)):
            slot.read_dtype = self.root_dtype
            if self.mode == 0:
                root = slot.computepower(4, self.eps)
            else:
                stat, _ = slot.dequantize()
                root = newton_root(stat.clone(), 4, self.eps, v0s[i])
            slot.read_dtype = torch.float32
            prec.put(root.float())
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
