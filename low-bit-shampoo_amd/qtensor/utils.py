"""Stateful quantized square matrices used by the Shampoo preconditioners.

Three holders with the constructor signatures, attribute names and method names of the
reference's qtensor/utils.py (QTensor :7-61, QTensorDiagReal :64-121, QTensorSVDFast
:124-236), so optimizer code written against the reference keeps working:

  QTensor          packed codes + per-segment maxima
  QTensorDiagReal  the same, with the diagonal kept exactly in fp32
  QTensorSVDFast   a PSD statistic held as a quantized eigenvector matrix plus the smaller
                   half of its eigenvalues in fp32

With bits in (32, 16), or fewer than min_lowbit_size elements, a holder just keeps the
matrix in fp32 / bf16.
"""
import re
from pathlib import Path

import torch

import qtensor.functional as F


class _LowBitState:
    """Buffer bookkeeping shared by the three holders."""

    def _adopt_format(self, var, bits, name2qmap, code, blocksize, min_lowbit_size, dense=None):
        """Decides between dense and low-bit storage.  Returns True when low-bit."""
        self.bits = bits
        if bits in (32, 16) or var.numel() < min_lowbit_size:
            return False
        if bits not in (8, 4):
            raise ValueError(f'num of bits is not supported: {bits}')
        name2qmap[code] = name2qmap[code].to(var.device)
        self.name2qmap = name2qmap
        self.code = code
        self.blocksize = blocksize
        self.var_order = var.shape[0]
        return True

    @property
    def _table(self):
        return self.name2qmap[self.code]

    def _kw(self):
        return dict(code=self._table, order=self.var_order, blocksize=self.blocksize, bits=self.bits)

    def _follow_order(self, var, names):
        """A matrix of another order arrives: drop the old buffers so new ones get allocated."""
        if var.shape[0] != self.var_order:
            self.var_order = var.shape[0]
            self.var_dtype = var.dtype
            for n in names:
                setattr(self, n, None)

    def _move(self, device, names):
        if self.bits < 16:
            self.name2qmap[self.code] = self._table.to(device)
            for n in names:
                setattr(self, n, getattr(self, n).to(device))
        self.var = self.var.to(device)

    # ---- flat checkpoint form (no counterpart in the reference, which pickles the holder objects:
    # optimizers/shampoo2.py:311-317 with qtensor/utils.py:57-61) ---------------------------------
    _lowbit_tensors = ()                            # side buffers of the low-bit form, per holder class

    def state_dict(self):
        """Plain tensors and numbers only: 'bits', 'var' (uint8 codes, first element of a pair in the high
        nibble, or the matrix itself for bits 16 / 32) and, when low-bit, 'order', 'dtype' and the side buffers
        ('absmax' fp32 [order * ceil(order / blocksize)], 'diag' fp32 [order] for the exact-diagonal form)."""
        out = {"bits": int(self.bits), "var": self.var}
        if self.bits < 16:
            out["order"] = int(self.var_order)
            out["dtype"] = str(self.var_dtype).replace("torch.", "")
            for name in self._lowbit_tensors:
                out[name] = getattr(self, name)
        return out

    def load_state_dict(self, sd):
        """Takes what state_dict() wrote into a holder constructed with the same arguments."""
        if int(sd["bits"]) != int(self.bits):
            raise ValueError(f"checkpointed holder has {int(sd['bits'])} bits, this one {self.bits}")
        device = self.var.device
        if self.bits >= 16:
            self.var = sd["var"].to(device=device, dtype=self.var.dtype).clone()
            return
        self.var_order = int(sd["order"])
        self.var_dtype = getattr(torch, sd["dtype"])
        self.var = sd["var"].to(device).clone()
        for name in self._lowbit_tensors:
            setattr(self, name, sd[name].to(device).clone())


class QTensor(_LowBitState):
    _lowbit_tensors = ("absmax",)

    def __init__(self, var, bits=32, name2qmap={}, code='', blocksize=2048, min_lowbit_size=4096):
        if self._adopt_format(var, bits, name2qmap, code, blocksize, min_lowbit_size):
            self.var_dtype = var.dtype
            self.var, self.absmax = F.quantize_blockwise(var, **self._kw())
        elif bits == 16:
            self.var, self.bits = var.bfloat16(), 16
        else:
            self.var, self.bits = var.float(), 32

    def quantize(self, var):
        if self.bits >= 16:
            self.var = var.to(self.var.dtype)
            return
        self._follow_order(var, ("var", "absmax"))
        self.var, self.absmax = F.quantize_blockwise(var.contiguous(), absmax=self.absmax, out=self.var, **self._kw())

    def dequantize(self):
        if self.bits >= 16:
            return self.var
        return F.dequantize_blockwise(self.var, absmax=self.absmax, outdtype=self.var_dtype, **self._kw())

    def set_device(self, device):
        self._move(device, ("absmax",))


class QTensorDiagReal(_LowBitState):
    _lowbit_tensors = ("absmax", "diag")

    def __init__(self, var, bits=32, name2qmap={}, code='', blocksize=2048, min_lowbit_size=4096):
        if self._adopt_format(var, bits, name2qmap, code, blocksize, min_lowbit_size):
            self.var_dtype = var.dtype
            self.var, self.absmax, self.diag = F.quantize_blockwise_diagreal(var, **self._kw())
        elif bits == 16:
            self.var, self.bits = var.bfloat16(), 16
        else:
            self.var, self.bits = var.float(), 32

    def quantize(self, var):
        if self.bits >= 16:
            self.var = var.to(self.var.dtype)
            return
        self._follow_order(var, ("var", "absmax", "diag"))
        self.var, self.absmax, self.diag = F.quantize_blockwise_diagreal(
            var.contiguous(), absmax=self.absmax, diag=self.diag, out=self.var, **self._kw())

    def dequantize(self):
        if self.bits >= 16:
            return self.var
        return F.dequantize_blockwise_diagreal(self.var, absmax=self.absmax, diag=self.diag,
                                               outdtype=self.var_dtype, **self._kw())

    def set_device(self, device):
        self._move(device, ("absmax", "diag"))


def _orthonormal_basis(Y):
    """Q factor of a QR factorisation of Y (reference: torch.linalg.qr at qtensor/utils.py:157): on a
    GPU through the batched Cholesky QR of qtensor.fused (the vendor's Householder routine takes
    about 20 ms for one 1024 x 1024 matrix), which gives the same Q up to the signs of its columns."""
    if Y.is_cuda and F.lib is not None and Y.dtype == torch.float32 and Y.dim() == 2 and Y.shape[0] == Y.shape[1]:
        from qtensor import fused
        return fused.cholesky_qr(Y.unsqueeze(0).contiguous())[0][0]
    return torch.linalg.qr(Y)[0]


class QTensorSVDFast(_LowBitState):
    """PSD statistic L ~ V_keep^T diag(Svalue) V_keep.

    `var` holds the (quantized) matrix Vt whose ROWS are approximate eigenvectors of L;
    Svalue / keep_indices are the smaller half of the Rayleigh quotients and the rows they
    belong to; max_eigenvalue is the largest quotient (used to scale the ridge term).
    rect_t1 / rect_t2 Bjorck steps re-orthonormalise Vt after dequantization."""
    _lowbit_tensors = ("absmax",)

    def state_dict(self):
        """As the other holders ('var' = the basis Vt), plus 'Svalue' fp32 [n/2], 'keep_indices' int64 [n/2]
        and 'max_eigenvalue' (fp32 scalar)."""
        out = super().state_dict()
        out.update(Svalue=self.Svalue, keep_indices=self.keep_indices, max_eigenvalue=self.max_eigenvalue,
                   log_written=bool(self._log_written))
        return out

    def load_state_dict(self, sd):
        super().load_state_dict(sd)
        device = self.var.device
        self.Svalue = sd["Svalue"].to(device).clone()
        self.keep_indices = sd["keep_indices"].to(device=device, dtype=torch.int64).clone()
        self.max_eigenvalue = sd["max_eigenvalue"].to(device).clone()
        self._log_written = bool(sd.get("log_written", False))

    def __init__(self, var, bits=32, name2qmap={}, code='', blocksize=2048, min_lowbit_size=4096,
                 rect_t1=1, rect_t2=4, log_prefix=None):
        self.rect_t1 = rect_t1
        self.rect_t2 = rect_t2
        self.log_prefix = log_prefix
        self._log_written = False

        n = var.shape[0]
        basis = torch.eye(n, device=var.device)
        start = var[0][0] * basis.diag()
        self.keep_indices = torch.arange(n, device=var.device, dtype=torch.int64)[:max(1, n // 2)]
        self.Svalue = start[self.keep_indices].clone()
        self.max_eigenvalue = start.max().clone()

        if self._adopt_format(var, bits, name2qmap, code, blocksize, min_lowbit_size):
            self.var_dtype = basis.dtype
            self.var, self.absmax = F.quantize_blockwise(basis, **self._kw())
        else:
            self.var, self.bits = basis, 32

    def _basis(self):
        return F.dequantize_blockwise(self.var, absmax=self.absmax, outdtype=self.var_dtype, **self._kw())

    def quantize(self, var, Vt=None):
        """One subspace-iteration step: orthonormalise L Vt^T by QR, take Rayleigh quotients,
        remember the smaller half, store the new basis (as rows)."""
        L = var.float()
        from qtensor import fused
        if fused.on_matrix_cores(L, Vt) and L.dim() == 2:
            # the same products on the matrix cores; the Rayleigh quotients diag(V^T (L V)) without the product
            V = _orthonormal_basis(fused.gemm(L, Vt, trans_b=True))
            quotients = (V * fused.gemm(L, V.contiguous())).sum(dim=0)
        else:
            V = _orthonormal_basis(L @ Vt.T.float())
            quotients = (V.T @ L @ V).diag()

        keep = max(1, quotients.numel() // 2)
        ascending, where = torch.sort(quotients)
        self.keep_indices = where[:keep].to(dtype=torch.int64)
        self.Svalue = ascending[:keep].to(var.dtype)
        dropped = ascending[keep:].to(var.dtype)
        self.max_eigenvalue = quotients.max().to(var.dtype)

        if self.bits >= 16:
            self.var = V.T.contiguous()
        elif V.is_cuda and V.dtype == torch.float32 and V.is_contiguous() and self.var_order % self.blocksize == 0:
            # the quantizer reads V as it lies and writes the codes of V.T (no transposed copy)
            from qtensor import fused
            fused.quantize_stack(V.unsqueeze(0), fused.Quantized.from_holder(self), transposed=True)
        else:
            F.quantize_blockwise(V.T.contiguous(), absmax=self.absmax, out=self.var, **self._kw())

        if self.log_prefix and not self._log_written:
            self._dump_spectrum(self.Svalue.detach().cpu(), dropped.detach().cpu())

    def _dump_spectrum(self, kept, dropped):
        # One-off CSV of the kept then dropped quotients, as the reference writes on the
        # first update of each statistic (qtensor/utils.py:173-189 of the reference).
        folder = Path("logs")
        folder.mkdir(parents=True, exist_ok=True)
        name = re.sub(r"[^A-Za-z0-9_.-]", "_", self.log_prefix)
        with open(folder / f"eigenvalues_{name}.csv", "w", encoding="utf-8") as fh:
            fh.write("rank,value\n")
            for rank, val in enumerate(list(kept) + list(dropped), start=1):
                fh.write(f"{rank},{float(val)}\n")
        self._log_written = True

    def dequantize(self):
        """Returns (V_keep^T diag(Svalue) V_keep, Vt)."""
        from qtensor import fused
        if self.bits < 16:
            Vt = self._basis()
            own = fused.on_matrix_cores(Vt)
            for _ in range(self.rect_t1):
                if own:
                    Vt = fused.gemm(fused.gemm(Vt, Vt, trans_b=True, symmetric=True), Vt, addend=Vt, alpha=-0.5, beta=1.5)
                else:
                    Vt = 1.5 * Vt - 0.5 * Vt @ Vt.T @ Vt
        else:
            Vt = self.var
        rows = Vt[self.keep_indices.to(device=Vt.device)]
        weights = self.Svalue.to(device=Vt.device, dtype=Vt.dtype)
        if fused.on_matrix_cores(rows):
            return fused.gemm(rows * weights.unsqueeze(1), rows, trans_a=True, symmetric=True), Vt
        return rows.T @ weights.diag() @ rows, Vt

    def computepower(self, exp, ridge_epsilon=1e-6):
        low = self.bits < 16
        return F.compute_power(
            self._basis() if low else self.var, self.Svalue, exp,
            iter_count=self.rect_t2 if low else 0, ridge_epsilon=ridge_epsilon,
            indices=self.keep_indices, max_eigen=self.max_eigenvalue)

    def set_device(self, device):
        self._move(device, ("absmax",))
        self.Svalue = self.Svalue.to(device)
        self.keep_indices = self.keep_indices.to(device)
        self.max_eigenvalue = self.max_eigenvalue.to(device)
