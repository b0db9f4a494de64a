"""Batched fp32 products on the MI355X matrix cores with the (de)quantization fused in.

No counterpart module exists in the reference: there these steps are separate torch calls per
matrix -- dequantize, then `@` (optimizers/shampoo2.py:255-268, shampoo1.py:164-178, 224-237)
and the matmuls of optimizers/matrix_functions.py:127-140.  Every function here takes GPU
tensors only and launches libqtensor_hip.so's qtensor_hip_gemm on torch's current stream.
"""
import ctypes as ct
from typing import Optional, Sequence

import numpy as np
import torch
from torch import Tensor

import qtensor.functional as F

DENSE, DENSE_T, QUANT4, QUANT8 = 0, 1, 2, 3
EPI_STORE, EPI_AXPBY_DENSE, EPI_AXPBY_QUANT4, EPI_AXPBY_QUANT8, EPI_NEWTON, EPI_REQUANT4, EPI_REQUANT8 = 0, 1, 2, 3, 4, 5, 6


class BatchPtr(ct.Structure):
    _fields_ = [("base", ct.c_void_p), ("list", ct.c_void_p), ("stride", ct.c_longlong)]


class QuantRef(ct.Structure):
    _fields_ = [("codes", BatchPtr), ("absmax", BatchPtr), ("diag", BatchPtr), ("order", ct.c_int),
                ("bs_shift", ct.c_int)]


class GemmArgs(ct.Structure):
    _fields_ = [("M_", ct.c_int), ("N_", ct.c_int), ("K_", ct.c_int),
                ("A", BatchPtr), ("lda", ct.c_int),
                ("B", BatchPtr), ("ldb", ct.c_int),
                ("Aq", QuantRef), ("Bq", QuantRef),
                ("C", BatchPtr), ("ldc", ct.c_int),
                ("alpha", ct.c_float), ("beta", ct.c_float),
                ("E", BatchPtr), ("lde", ct.c_int),
                ("Eq", QuantRef),
                ("T", BatchPtr), ("ldt", ct.c_int),
                ("newton_w", ct.c_float),
                ("err", ct.c_void_p), ("skip", ct.c_void_p), ("code", ct.c_void_p), ("symmetric", ct.c_int),
                ("workspace", ct.c_void_p), ("workspace_floats", ct.c_longlong), ("split_k_", ct.c_int),
                ("batch_count_", ct.c_int), ("stream_per_", ct.c_int), ("stream_lcm_", ct.c_int),
                ("batch_inner", ct.c_int), ("inner_a", ct.c_longlong), ("inner_b", ct.c_longlong),
                ("inner_c", ct.c_longlong), ("inner_e", ct.c_longlong), ("triangular", ct.c_int), ("pipe", ct.c_int)]


class GemmDesc(ct.Structure):
    _fields_ = [("M", ct.c_int), ("N", ct.c_int), ("K", ct.c_int), ("batch", ct.c_int),
                ("kind_a", ct.c_int), ("kind_b", ct.c_int), ("epilogue", ct.c_int), ("args", GemmArgs)]


if F.lib is not None:
    F.lib.qtensor_hip_gemm_pipe.restype = ct.c_int
    F.lib.qtensor_hip_gemm_pipe.argtypes = [ct.c_int]
    F.lib.qtensor_hip_gemm.restype = None
    F.lib.qtensor_hip_gemm.argtypes = [ct.POINTER(GemmDesc), ct.c_void_p]


class Quantized:
    """A batch of equally sized quantized square matrices held in stacked buffers.

    codes [batch, ceil(order*order*bits/8)] uint8, absmax [batch, order*ceil(order/blocksize)] fp32,
    diag [batch, order] fp32 or None, all contiguous on one GPU.  Entry b is exactly what
    quantize_blockwise(_diagreal) writes for one matrix.  `flat`: the blocksize divides the order, so a
    matrix is one stream of whole segments -- the layout the products read directly (as an operand or an
    addend); stacks of any other order go through quantize_stack / dequantize_stack only."""

    def __init__(self, codes: Tensor, absmax: Tensor, diag: Optional[Tensor], order: int, blocksize: int,
                 bits: int, code: Tensor):
        self.codes, self.absmax, self.diag = codes, absmax, diag
        self.order, self.blocksize, self.bits, self.code = order, blocksize, bits, code
        self.batch = codes.shape[0] if codes.dim() == 2 else 1
        self.flat = order % blocksize == 0

    def rows(self, first: int, count: int) -> "Quantized":
        """The entries first .. first + count - 1 of the stack, as views."""
        return Quantized(self.codes[first:first + count], self.absmax[first:first + count],
                         None if self.diag is None else self.diag[first:first + count], self.order, self.blocksize,
                         self.bits, self.code)

    def select(self, index: Tensor) -> "Quantized":
        """A copy of the entries index (int64 GPU vector)."""
        return Quantized(self.codes.index_select(0, index), self.absmax.index_select(0, index),
                         None if self.diag is None else self.diag.index_select(0, index), self.order, self.blocksize,
                         self.bits, self.code)

    def put(self, index: Tensor, other: "Quantized") -> None:
        """Entries index of this stack = the entries of other, in order."""
        self.codes.index_copy_(0, index, other.codes)
        self.absmax.index_copy_(0, index, other.absmax)
        if self.diag is not None:
            self.diag.index_copy_(0, index, other.diag)

    @classmethod
    def from_holder(cls, h) -> "Quantized":
        """View of one qtensor.utils holder (QTensor or QTensorDiagReal in low-bit mode)."""
        return cls(h.var.view(1, -1), h.absmax.view(1, -1), None if getattr(h, "diag", None) is None else h.diag.view(1, -1),
                   h.var_order, h.blocksize, h.bits, h.name2qmap[h.code])

    def ref(self) -> QuantRef:
        if not self.flat:
            raise ValueError("the products read quantized matrices whose order the blocksize divides; dequantize this stack first")
        q = QuantRef()
        q.codes = BatchPtr(self.codes.data_ptr(), None, self.codes.stride(0) if self.codes.dim() == 2 else 0)
        q.absmax = BatchPtr(self.absmax.data_ptr(), None, self.absmax.stride(0) if self.absmax.dim() == 2 else 0)
        if self.diag is not None:
            q.diag = BatchPtr(self.diag.data_ptr(), None, self.diag.stride(0) if self.diag.dim() == 2 else 0)
        q.order = self.order
        q.bs_shift = self.blocksize.bit_length() - 1
        return q

    @property
    def kind(self) -> int:
        return QUANT4 if self.bits == 4 else QUANT8


class PtrList:
    """A batch of dense fp32 matrices given by a device array of addresses (int64 [batch]), all of
    shape rows x cols with leading dimension ld (default cols).  Lets a caller choose per batch
    entry, on the device, which buffer an operand comes from or a result goes to."""

    def __init__(self, ptrs: Tensor, shape, ld: Optional[int] = None):
        if ptrs.dtype != torch.int64 or not ptrs.is_cuda or ptrs.dim() != 1 or ptrs.numel() != shape[0]:
            raise ValueError("PtrList needs an int64 GPU vector with one address per batch entry")
        self.ptrs, self.shape, self.ld = ptrs.contiguous(), tuple(shape), (shape[2] if ld is None else ld)
        self.device = ptrs.device

    def dim(self):
        return 3


def _dense(t):
    """(BatchPtr, leading dimension, batch, rows, cols) of a [rows, cols] or [batch, rows, cols] fp32 tensor whose
    last dimension is contiguous, or of a PtrList."""
    if isinstance(t, PtrList):
        return BatchPtr(None, t.ptrs.data_ptr(), 0), t.ld, t.shape[0], t.shape[1], t.shape[2]
    if t.dtype != torch.float32 or not t.is_cuda:
        raise ValueError("fused products take fp32 GPU tensors")
    if t.dim() == 2:
        t = t.unsqueeze(0)
    if t.dim() != 3 or t.stride(2) != 1:
        raise ValueError("expected [rows, cols] or [batch, rows, cols] with a contiguous last dimension")
    return BatchPtr(t.data_ptr(), None, t.stride(0)), t.stride(1), t.shape[0], t.shape[1], t.shape[2]


_WORKSPACE_FLOATS = 1 << 24     # 64 MiB: the most a product that is cut along k gets for its partial products


def _workspace(device: torch.device, floats: int) -> Tensor:
    """fp32 scratch for one product that may be cut along k: taken from torch's allocator for the call and handed
    back with it (the allocator keeps it for the stream it was used on), so that nothing is held between steps."""
    return torch.empty(min(_WORKSPACE_FLOATS, floats), dtype=torch.float32, device=device)


def _launch(desc: GemmDesc, device: torch.device) -> None:
    if F.lib is None:
        raise RuntimeError("libqtensor_hip.so is not available")
    F._call(lambda d, s: F.lib.qtensor_hip_gemm(d, s), device, ct.byref(desc))


def gemm_pipe(mode: Optional[str] = None) -> str:
    """Which matrix pipe multiplies (dense and quantized operands alike), for the whole process: "f32" (fp32 MFMA) or "split"
    (operands split into three bf16 pieces, six bf16 products per fp32 product, fp32 accumulation: fp32-grade
    results at a multiple of the fp32 pipe's rate).  Sets the mode when given; returns the one in force before."""
    if F.lib is None:
        raise RuntimeError("libqtensor_hip.so is not available")
    names = ("f32", "split")
    if mode is not None and mode not in names:
        raise ValueError(f"mode must be one of {names}")
    return names[F.lib.qtensor_hip_gemm_pipe(-1 if mode is None else names.index(mode))]


_PIPES = {None: 0, "f32": 1, "split": 2}


def gemm(A, B, *, trans_a=False, trans_b=False, out: Optional[Tensor] = None, alpha=1.0, beta=0.0,
         addend=None, newton=None, skip: Optional[Tensor] = None, symmetric: bool = False,
         upper_a: bool = False, upper_b: bool = False, requantize: bool = False, pipe: Optional[str] = None):
    """out[b] = epilogue(op(A[b]) @ op(B[b])).

    A, B: fp32 tensors ([m,k] / [batch,m,k]; with trans_x the stored matrix is the transpose; trans_a together
    with trans_b is not built: that product is the transpose of B A) or a `Quantized` (square; then the other
    operand must be dense).
    addend: None, a dense tensor E or a `Quantized` E: out = beta*E + alpha*product.
    newton: None or (T_out, w, err): also writes T_out = (1-w) I + w*product and folds
    max|product - I| into err[b] (fp32 [batch], zeroed by the caller).
    skip: optional int32 [batch]; entries with a nonzero flag are not touched.
    symmetric: the caller knows the product to be symmetric (a Gram matrix, a product of commuting
    symmetric matrices): only the tiles on and above the diagonal are multiplied out and mirrored,
    which halves the work; the result is then symmetric bit for bit outside the diagonal tiles.
    requantize (with a `Quantized` addend of blocksize 64): beta*E + alpha*product is encoded straight back
    into E's buffers (codes, maxima, exact diagonal) -- bit-identical to writing it out and quantizing it, but
    the fp32 matrix never reaches memory; returns E.
    upper_a / upper_b: op(A) / op(B) is upper triangular (zero below the diagonal, square in its k
    index, dense): the part of the k range where it is zero is skipped.
    pipe: None (the process-wide choice, gemm_pipe), "f32" or "split" for this product alone."""
    d = GemmDesc()
    a = d.args
    if pipe not in _PIPES:
        raise ValueError('pipe must be None, "f32" or "split"')
    a.pipe = _PIPES[pipe]
    dev = None
    code = None
    if isinstance(A, Quantized):
        if trans_a:
            raise ValueError("a quantized operand cannot be transposed")
        d.kind_a, a.Aq, batch_a, m, k = A.kind, A.ref(), A.batch, A.order, A.order
        dev, code = A.codes.device, A.code
    else:
        a.A, a.lda, batch_a, r, c = _dense(A)
        m, k = (c, r) if trans_a else (r, c)
        d.kind_a = DENSE_T if trans_a else DENSE
        dev = A.device
    if isinstance(B, Quantized):
        if trans_b:
            raise ValueError("a quantized operand cannot be transposed")
        d.kind_b, a.Bq, batch_b, k2, n = B.kind, B.ref(), B.batch, B.order, B.order
        code = B.code
    else:
        a.B, a.ldb, batch_b, r, c = _dense(B)
        k2, n = (c, r) if trans_b else (r, c)
        d.kind_b = DENSE_T if trans_b else DENSE
    if k != k2:
        raise ValueError(f"inner dimensions differ: {k} vs {k2}")
    if batch_a != batch_b:
        raise ValueError(f"batch sizes differ: {batch_a} vs {batch_b}")
    batch = batch_a
    if requantize:
        if not isinstance(addend, Quantized) or addend.blocksize != 64 or out is not None or newton is not None:
            raise ValueError("requantize needs a quantized addend of blocksize 64 and takes no other output")
    else:
        if out is None:
            out = torch.empty((batch, m, n), device=dev, dtype=torch.float32)
            squeeze = (not isinstance(A, Quantized) and A.dim() == 2) or (not isinstance(B, Quantized) and B.dim() == 2)
            if squeeze and batch == 1:
                out = out[0]
        a.C, a.ldc, batch_c, mc, nc = _dense(out)
        if (batch_c, mc, nc) != (batch, m, n):
            raise ValueError(f"out has shape {tuple(out.shape)}, expected batch {batch} x {m} x {n}")
    d.M, d.N, d.K, d.batch = m, n, k, batch
    d.epilogue = EPI_STORE
    a.alpha, a.beta = alpha, beta
    if addend is not None:
        if isinstance(addend, Quantized):
            if addend.batch != batch or addend.order != m or m != n:
                raise ValueError("quantized addend must match the batch and be m x m")
            a.Eq = addend.ref()
            d.epilogue = EPI_AXPBY_QUANT4 if addend.bits == 4 else EPI_AXPBY_QUANT8
            if requantize:
                d.epilogue = EPI_REQUANT4 if addend.bits == 4 else EPI_REQUANT8
            code = addend.code
        else:
            a.E, a.lde, be, me, ne = _dense(addend)
            if (be, me, ne) != (batch, m, n):
                raise ValueError("dense addend must have the shape of the result")
            d.epilogue = EPI_AXPBY_DENSE
    keep = [out]
    if newton is not None:
        if addend is not None:
            raise ValueError("the Newton epilogue takes no addend")
        t_out, w, err = newton
        a.T, a.ldt, bt, mt, nt = _dense(t_out)
        if (bt, mt, nt) != (batch, m, n) or err.numel() != batch or err.dtype != torch.float32:
            raise ValueError("Newton outputs must match the result")
        a.newton_w = w
        a.err = err.data_ptr()
        d.epilogue = EPI_NEWTON
    if skip is not None:
        if skip.dtype != torch.int32 or skip.numel() != batch:
            raise ValueError("skip must be int32 [batch]")
        a.skip = skip.data_ptr()
    if code is not None:
        a.code = code.data_ptr()
    if symmetric:
        if m != n or isinstance(A, Quantized) or isinstance(B, Quantized):
            raise ValueError("symmetric products are square with dense operands")
        a.symmetric = 1
    if upper_a or upper_b:
        if symmetric or isinstance(A, Quantized) or isinstance(B, Quantized) or (upper_a and m != k) or (upper_b and n != k):
            raise ValueError("triangular operands are dense and square, in a product that is not marked symmetric")
        a.triangular = (1 if upper_a else 0) | (2 if upper_b else 0)
    if d.epilogue == EPI_STORE and not symmetric and k >= 256 and batch * m * n <= _WORKSPACE_FLOATS // 2:
        # few output tiles, long k: the library may cut k into up to eight slices per tile, or -- with a quantized
        # operand -- deal runs of k tiles out over two workgroups per compute unit (a 128 x 128 square per run and tile)
        tiles = batch * (-(-m // 128)) * (-(-n // 128))
        quantized = isinstance(A, Quantized) or isinstance(B, Quantized)
        scratch = _workspace(dev, max(8 * batch * m * n, (tiles + 520) * 128 * 128 if quantized and tiles < 1024 else 0))
        a.workspace, a.workspace_floats = scratch.data_ptr(), scratch.numel()
        keep.append(scratch)
    _launch(d, dev)
    return addend if requantize else out


def on_matrix_cores(*tensors) -> bool:
    """Whether a product of these tensors can go through gemm(): fp32 GPU tensors with a contiguous last dimension
    (and the library there)."""
    return F.lib is not None and all(t.is_cuda and t.dtype == torch.float32 and t.dim() in (2, 3) and t.stride(-1) == 1
                                     and t.numel() > 0 for t in tensors)


if F.lib is not None:
    F.lib.qtensor_hip_matvec_batched.restype = None
    F.lib.qtensor_hip_matvec_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_void_p]


def matvec(mats: Tensor, v: Tensor) -> Tensor:
    """[B, n]: mats[b] @ v[b] for a contiguous fp32 GPU stack [B, n, n] and vectors [B, n], one launch, fixed
    summation order (the reference: torch.mv per matrix, optimizers/matrix_functions.py:42)."""
    B, n, _ = mats.shape
    _stack(mats, "mats", (B, n, n)), _stack(v, "v", (B, n))
    out = torch.empty(B, n, device=mats.device)
    F._call(F.lib.qtensor_hip_matvec_batched, mats.device, mats.data_ptr(), v.data_ptr(), out.data_ptr(), n, B)
    return out


def precondition(G: Tensor, left, right, out: Optional[Tensor] = None) -> Tensor:
    """deq(left) @ G @ deq(right) with both factors expanded inside the products.
    left / right: `Quantized` or dense fp32 matrices."""
    tmp = gemm(left, G)
    return gemm(tmp, right, out=out)


def gram(G: Tensor, axis: int, *, stat=None, beta=0.0, alpha=1.0, out: Optional[Tensor] = None) -> Tensor:
    """axis 0: G @ G.T, axis 1: G.T @ G; with `stat` (dense or `Quantized`) returns
    beta * stat + alpha * that product, i.e. the Shampoo statistics update in one launch."""
    if axis == 0:
        return gemm(G, G, trans_b=True, addend=stat, alpha=alpha, beta=beta, out=out, symmetric=True)
    return gemm(G, G, trans_a=True, addend=stat, alpha=alpha, beta=beta, out=out, symmetric=True)


# --------------------------------------------------------------------------- stacks of matrices
if F.lib is not None:
    F.lib.qtensor_hip_quantize_batched.restype = None
    F.lib.qtensor_hip_quantize_batched.argtypes = [ct.c_void_p, ct.c_int, ct.c_void_p, ct.c_int, ct.c_int, ct.c_int,
                                                   ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_void_p]
    F.lib.qtensor_hip_quantize_transposed_batched.restype = None
    F.lib.qtensor_hip_quantize_transposed_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_int,
                                                              ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_void_p]
    F.lib.qtensor_hip_dequantize_batched.restype = None
    F.lib.qtensor_hip_dequantize_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_int, ct.c_void_p,
                                                     ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_void_p]


def empty_quantized(batch: int, order: int, blocksize: int, bits: int, code: Tensor, diagreal: bool) -> Quantized:
    """Uninitialised stacked buffers for `batch` matrices of the given order (any order: a last segment of a
    row may be shorter, and the codes of an odd order are padded to a whole byte per matrix, as in the
    single-matrix format)."""
    dev = code.device
    codes = torch.empty(batch, -(-(order * order * bits) // 8), dtype=torch.uint8, device=dev)
    absmax = torch.empty(batch, order * (-(-order // blocksize)), dtype=torch.float32, device=dev)
    diag = torch.empty(batch, order, dtype=torch.float32, device=dev) if diagreal else None
    return Quantized(codes, absmax, diag, order, blocksize, bits, code)


def quantize_stack(mats: Tensor, q: Quantized, transposed: bool = False) -> Quantized:
    """Quantize the contiguous stack mats [batch, order, order] (fp32 or bf16) into q's buffers in one
    launch; entry b equals quantize_blockwise(_diagreal)(mats[b]) -- of mats[b].T with transposed=True,
    which reads the stack as it lies (one kernel turns 64-column tiles around on the way; reference:
    V.T.contiguous() before the quantizer, qtensor/utils.py:169-170) when the form is plain, the input
    fp32, and the blocksize is 64, 128 or 256 and divides an order that is a multiple of 64."""
    if F.lib is None:
        raise RuntimeError("libqtensor_hip.so is not available")
    if not mats.is_cuda or not mats.is_contiguous() or mats.shape != (q.batch, q.order, q.order):
        raise ValueError(f"expected a contiguous GPU stack of shape {(q.batch, q.order, q.order)}")
    slot = F._dtype_slot(mats.dtype, "mats")
    for t in (q.codes, q.absmax) + ((q.diag,) if q.diag is not None else ()):
        if not t.is_contiguous():
            raise ValueError("stacked quantized buffers must be contiguous")
    if q.batch > 65535 and not q.flat:
        for first in range(0, q.batch, 65535):
            quantize_stack(mats[first:first + 65535], q.rows(first, min(65535, q.batch - first)), transposed)
        return q
    if transposed:
        if (q.diag is None and mats.dtype == torch.float32 and q.blocksize in (64, 128, 256)
                and q.order % q.blocksize == 0 and q.order % 64 == 0):
            F._call(F.lib.qtensor_hip_quantize_transposed_batched, mats.device, mats.data_ptr(), q.code.data_ptr(), q.bits,
                    q.order, q.batch, q.absmax.data_ptr(), q.codes.data_ptr(), q.blocksize)
            return q
        mats = mats.transpose(1, 2).contiguous()
    F._call(F.lib.qtensor_hip_quantize_batched, mats.device, mats.data_ptr(), slot, q.code.data_ptr(), q.bits, q.order,
            q.batch, q.absmax.data_ptr(), None if q.diag is None else q.diag.data_ptr(), q.codes.data_ptr(), q.blocksize)
    return q


def dequantize_stack(q: Quantized, out: Optional[Tensor] = None, outdtype=torch.float32) -> Tensor:
    """[batch, order, order] stack of dequantized matrices in one launch."""
    if F.lib is None:
        raise RuntimeError("libqtensor_hip.so is not available")
    if out is None:
        out = torch.empty(q.batch, q.order, q.order, dtype=outdtype, device=q.codes.device)
    if not out.is_contiguous() or out.shape != (q.batch, q.order, q.order):
        raise ValueError(f"out must be a contiguous stack of shape {(q.batch, q.order, q.order)}")
    slot = F._dtype_slot(out.dtype, "out")
    if q.batch > 65535 and not q.flat:
        for first in range(0, q.batch, 65535):
            dequantize_stack(q.rows(first, min(65535, q.batch - first)), out[first:first + 65535])
        return out
    F._call(F.lib.qtensor_hip_dequantize_batched, out.device, q.codes.data_ptr(), q.code.data_ptr(), q.bits, q.order,
            q.batch, q.absmax.data_ptr(), None if q.diag is None else q.diag.data_ptr(), out.data_ptr(), slot, q.blocksize)
    return out


class DenseStack:
    """A stack of square matrices [batch, order, order] kept as it is (fp32), with the surface of `Quantized`
    that the batched step drivers use -- for orders with fewer than min_lowbit_size elements and for
    prec_bits = 32, where the reference's holders keep the matrix itself (qtensor/utils.py:11-17, 68-74)."""
    flat = False
    bits = 32
    diag = None

    def __init__(self, data: Tensor):
        if data.dim() != 3 or data.shape[1] != data.shape[2] or data.dtype != torch.float32:
            raise ValueError("DenseStack takes an fp32 stack [batch, order, order]")
        self.data = data
        self.batch, self.order = data.shape[0], data.shape[1]

    def rows(self, first: int, count: int) -> "DenseStack":
        return DenseStack(self.data[first:first + count])

    def select(self, index: Tensor) -> "DenseStack":
        return DenseStack(self.data.index_select(0, index))

    def put(self, index: Tensor, other: "DenseStack") -> None:
        self.data.index_copy_(0, index, other.data)


def load_stack(q) -> Tensor:
    """fp32 [batch, order, order] of a `Quantized` (a new tensor) or a `DenseStack` (its own tensor, no copy)."""
    return q.data if isinstance(q, DenseStack) else dequantize_stack(q)


def store_stack(mats: Tensor, q, transposed: bool = False):
    """Inverse of load_stack: mats (their transposes with transposed=True) into q's buffers."""
    if isinstance(q, DenseStack):
        src = mats.transpose(1, 2) if transposed else mats
        if transposed or src.data_ptr() != q.data.data_ptr():
            q.data.copy_(src.contiguous() if transposed else src)
        return q
    return quantize_stack(mats.contiguous(), q, transposed)


# --------------------------------------------------------------------------- Cholesky QR pieces
if F.lib is not None:
    F.lib.qtensor_hip_cholesky_upper_floor_batched.restype = None
    F.lib.qtensor_hip_cholesky_upper_floor_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_int,
                                                               ct.c_int, ct.c_float, ct.c_void_p]
    F.lib.qtensor_hip_block_gram_schmidt_width.restype = ct.c_int
    F.lib.qtensor_hip_block_gram_schmidt_width.argtypes = []
    F.lib.qtensor_hip_block_gram_schmidt_batched.restype = None
    F.lib.qtensor_hip_block_gram_schmidt_batched.argtypes = [ct.c_void_p] * 7 + [ct.c_int, ct.c_int, ct.c_float, ct.c_float, ct.c_void_p]
    F.lib.qtensor_hip_block_gram_schmidt_replacing_batched.restype = None
    F.lib.qtensor_hip_block_gram_schmidt_replacing_batched.argtypes = ([ct.c_void_p] * 7 +
                                                                       [ct.c_int, ct.c_int, ct.c_float, ct.c_float, ct.c_int, ct.c_void_p])
    F.lib.qtensor_hip_gram_deviation_batched.restype = None
    F.lib.qtensor_hip_gram_deviation_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_void_p]
    F.lib.qtensor_hip_column_dots_batched.restype = None
    F.lib.qtensor_hip_column_dots_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_void_p]
    F.lib.qtensor_hip_copy_flagged_batched.restype = None
    F.lib.qtensor_hip_copy_flagged_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_void_p]
    F.lib.qtensor_hip_solve_upper_right_batched.restype = None
    F.lib.qtensor_hip_solve_upper_right_batched.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_int,
                                                            ct.c_int, ct.c_int, ct.c_void_p]


def _stack(t: Tensor, name: str, shape=None) -> Tensor:
    if not t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous() or (shape is not None and tuple(t.shape) != tuple(shape)):
        raise ValueError(f"{name} must be a contiguous fp32 GPU tensor" + (f" of shape {tuple(shape)}" if shape else ""))
    return t


def cholesky_upper(gram: Tensor, u: Tensor, x: Tensor, info: Tensor, pivot_floor: float = 0.0) -> None:
    """gram [B, n, n] (destroyed) = U^T U: block rows of U into u, inverses of its 64 x 64 diagonal blocks
    into the diagonal blocks of x [B, n, n] (nothing else of x is written); info int32 [B] (zeroed by the
    caller): bit 0 = a non-positive or NaN pivot (factor meaningless), bit 1 = a pivot at or below
    pivot_floor > 0 was raised to it (with pivot_floor = 0 such a pivot sets bit 0)."""
    B, n, _ = gram.shape
    _stack(gram, "gram", (B, n, n)), _stack(u, "u", (B, n, n)), _stack(x, "x", (B, n, n))
    if info.dtype != torch.int32 or info.numel() != B or not info.is_cuda:
        raise ValueError("info must be an int32 GPU vector with one entry per matrix")
    F._call(F.lib.qtensor_hip_cholesky_upper_floor_batched, gram.device, gram.data_ptr(), u.data_ptr(), x.data_ptr(), info.data_ptr(),
            n, B, float(pivot_floor))


_COMPLETION = {}                 # (device index, order) -> fixed matrix of unit columns that stand in for null directions
NULL_COLUMN_NORM2 = 1e-11        # what a projection leaves of a unit column that depends on the earlier ones: rounding noise


def completion_columns(device: torch.device, n: int, true_n: int = None) -> Tensor:
    """[n, n] fixed pseudo-random unit columns (the same for every call): stand-ins for the columns of a
    rank-deficient matrix that are rounding noise once the columns before them are taken out.  true_n < n: the
    matrices are diag(Y, I) with Y of order true_n (orders padded to a multiple of 64) and so are the stand-ins,
    diag(F, I): a stand-in for a column of Y has nothing in the padding rows, or the part of Q that is handed back,
    its leading true_n x true_n block, would not be orthonormal."""
    true_n = n if true_n is None else true_n
    key = (device.index, n, true_n)
    if key not in _COMPLETION:
        gen = torch.Generator(device=device).manual_seed(0x5eed + n)
        r = torch.randn(n, n, device=device, generator=gen)
        if true_n < n:
            r[true_n:, :true_n] = 0.0
            r[:, true_n:] = 0.0
            r.diagonal()[true_n:] = 1.0
        _COMPLETION[key] = (r / torch.linalg.vector_norm(r, dim=0, keepdim=True)).contiguous()
    return _COMPLETION[key]


def block_gram_schmidt(q: Tensor, info: Tensor, pivot_floor: float = 2e-4, null_norm2: float = NULL_COLUMN_NORM2,
                       complete: bool = True, replace_dependent: bool = False, true_n: int = None) -> Tensor:
    """Orthonormalise the columns of every matrix of the stack q [B, n, n] (unit columns, n a multiple of 64)
    in place, left to right in panels of 64 columns: block Gram-Schmidt with reorthogonalisation, Cholesky QR
    inside a panel.  span(q[:, :, :k]) is kept for every k.  complete: columns that depend on the earlier ones
    up to rounding noise are replaced by fixed unit columns in general position (bit 2 of info[b]); info int32
    [B], zeroed by the caller, bits as in cholesky_upper.  replace_dependent (needs complete): a column that the
    first pass finds dependent inside its 64-column panel (pivot at or below pivot_floor) is replaced as well,
    instead of being handed to the second pass as it is -- for matrices of low numerical rank.  true_n < n: the
    matrices are diag(Y, I) with Y of order true_n, and the stand-in columns keep that form (completion_columns)."""
    B, n, _ = q.shape
    _stack(q, "q", (B, n, n))
    if info.dtype != torch.int32 or info.numel() != B or not info.is_cuda:
        raise ValueError("info must be an int32 GPU vector with one entry per matrix")
    w = torch.empty(B, n, F.lib.qtensor_hip_block_gram_schmidt_width(), device=q.device)
    small = torch.empty(3, B, 64, 64, device=q.device)
    fill = completion_columns(q.device, n, true_n) if complete else None
    if replace_dependent and fill is None:
        raise ValueError("replace_dependent needs complete=True")
    F._call(F.lib.qtensor_hip_block_gram_schmidt_replacing_batched, q.device, q.data_ptr(), w.data_ptr(), small[0].data_ptr(),
            small[1].data_ptr(), small[2].data_ptr(), None if fill is None else fill.data_ptr(), info.data_ptr(), n, B,
            float(pivot_floor), float(null_norm2), int(bool(replace_dependent)))
    return q


def gram_deviation(gram: Tensor) -> Tensor:
    """[B, 2]: max |G - I| and ||G - I||_F^2 of every matrix of the stack gram [B, n, n] (n a multiple of
    64), in one pass and a fixed summation order."""
    B, n, _ = gram.shape
    _stack(gram, "gram", (B, n, n))
    out = torch.empty(B, 2, device=gram.device)
    partial = torch.empty(B, 64, device=gram.device)
    F._call(F.lib.qtensor_hip_gram_deviation_batched, gram.device, gram.data_ptr(), partial.data_ptr(), out.data_ptr(), n, B)
    return out


def column_dots(a: Tensor, b: Tensor) -> Tensor:
    """[B, n]: sum_i a[:, i, j] * b[:, i, j] for two stacks [B, n, n] (n a multiple of 64) -- the diagonal of a^T b
    in one pass, fixed summation order."""
    B, n, _ = a.shape
    _stack(a, "a", (B, n, n)), _stack(b, "b", (B, n, n))
    out = torch.empty(B, n, device=a.device)
    F._call(F.lib.qtensor_hip_column_dots_batched, a.device, a.data_ptr(), b.data_ptr(), out.data_ptr(), n, B)
    return out


def copy_flagged(dst: Tensor, src: Tensor, flags: Tensor) -> Tensor:
    """dst[b] = src[b] for the matrices of the stacks [B, n, n] with flags[b] != 0 (int32 [B])."""
    B, n, _ = dst.shape
    _stack(dst, "dst", (B, n, n)), _stack(src, "src", (B, n, n))
    if flags.dtype != torch.int32 or flags.numel() != B or not flags.is_cuda:
        raise ValueError("flags must be an int32 GPU vector with one entry per matrix")
    F._call(F.lib.qtensor_hip_copy_flagged_batched, dst.device, dst.data_ptr(), src.data_ptr(), flags.data_ptr(), n, B)
    return dst


def solve_upper_right(q: Tensor, u: Tensor, x: Tensor, work: Tensor, out: Tensor) -> Tensor:
    """out = q U^-1 for q [B, rows, n] (rows <= n) with u, x from cholesky_upper; the inverted diagonal
    blocks of x (zero below them) are doubled up to 256 x 256 on the way; work: scratch [B, n, n]."""
    B, rows, n = q.shape
    _stack(q, "q"), _stack(u, "u", (B, n, n)), _stack(x, "x", (B, n, n)), _stack(work, "work", (B, n, n))
    _stack(out, "out", (B, rows, n))
    if out.data_ptr() == q.data_ptr():
        raise ValueError("out must not alias q")
    if rows > n:
        raise ValueError("the scratch area covers at most n rows")
    F._call(F.lib.qtensor_hip_solve_upper_right_batched, q.device, q.data_ptr(), u.data_ptr(), x.data_ptr(), work.data_ptr(),
            out.data_ptr(), rows, n, B)
    return out


_householder_qr = torch.linalg.qr
PIVOT_FLOOR = 2e-4               # a hundred times the rounding error of an fp32 Gram matrix of unit columns


class CholeskyQR:
    """Orthonormal Q [B, n, n] with span(Q[:, :, :k]) == span(Y[:, :, :k]) for every k (the Q factor
    of a QR factorisation with positive diagonal of R) for a whole stack.

    The work is done by one sweep of block Gram-Schmidt with reorthogonalisation over the column-scaled
    matrix (block_gram_schmidt: panels left to right, every panel has the finished columns taken out of it
    twice and is orthonormalised inside by Cholesky QR), which loses orthogonality only in proportion to
    fp32 rounding whatever the conditioning of Y.  What follows is a safety net of Cholesky QR rounds on the
    whole matrix --  G = Q^T Q,  U = chol(G),  Q <- Q U^-1,  every U upper triangular, so the nested spans
    survive -- for the few matrices the test after the sweep does not find orthonormal (typically a
    rank-deficient one whose last panel of stand-in columns is a little off): one round each.

    Rank-deficient Y (a statistic of order 768 fed by a 768 x 256 gradient block has rank 256 plus whatever
    its kept eigenpairs add): a column that depends on the ones before it is rounding noise once those are
    taken out, and the Q column it leads to is noise in any QR algorithm (Householder's included).  The
    sweep replaces such a column (shorter than sqrt(1e-11) after the first projection of a unit column) by a
    fixed unit column in general position, which is then orthogonalised like any other; columns with a real
    independent part, however small, are kept.  Inside the factorisations a pivot that is not above
    PIVOT_FLOOR takes its column out of that factorisation (cholesky_upper) instead of failing it.

    Once ||G - I||_F < 0.5 one Cholesky QR round makes Q orthonormal to fp32 rounding and the matrix leaves
    the working set without a further test.  A matrix that is farther than that and that two rounds in a row
    did not bring nearer than half of before (or a stack where every fourth matrix is that far right after
    the sweep) is of low numerical rank: rounds diverge there, and it is swept again from its original
    columns with every dependent column replaced by a stand-in (_repair).  Matrices that still are far three rounds after that, or after max_rounds, or whose
    factorisation meets a NaN, go through torch.linalg.qr.  Orders that are not a multiple of 64 are padded
    with an identity block (QR of diag(Y, I) is diag(Q, I)).

    The object is a small state machine so that several stacks can advance on their own streams while
    the host waits only once per round for all of them:  check() enqueues the orthonormality test,
    poll() reads its outcome (the only host synchronisation), advance() enqueues one round for the
    matrices still in the working set, result() returns (Q, number of matrices redone by the
    library).  All calls for one object must be made with the same current stream."""

    def __init__(self, Y, max_rounds=12, pivot_floor=PIVOT_FLOOR, tolerance=2e-5, sweep=True, replace_first=False,
                 remake=None, leave=()):
        """leave: matrices of the stack (their numbers) that the caller orthonormalises some other way: whatever the
        sweep makes of them is final here, they are neither tested nor polished.
        remake: optional callable, int64 GPU vector of matrix numbers -> those matrices of Y again.  With it Y is
        given up: its columns are scaled in place and it becomes the working set (one stack less held through the
        sweep); the few matrices whose original columns are needed again (_repair, the library fallback) are made anew."""
        if Y.dim() != 3 or Y.shape[1] != Y.shape[2] or Y.dtype != torch.float32 or not Y.is_cuda:
            raise ValueError("CholeskyQR takes an fp32 GPU stack [B, n, n]")
        B, self.true_n, _ = Y.shape
        n = -(-self.true_n // 64) * 64
        self.batch, self.n, self.device, self.remake = B, n, Y.device, remake
        self.leave = np.asarray(sorted(leave), dtype=np.int64)
        if n != self.true_n:
            Y = self._padded(Y)
        self.pivot_floor, self.tolerance, self.rounds_left = pivot_floor, tolerance, max_rounds
        scale = torch.linalg.vector_norm(Y, dim=1, keepdim=True).clamp_min(1e-30)
        if remake is not None and Y.is_contiguous():
            self.Y, self.Q = None, Y.div_(scale)
        else:
            self.Y, self.Q = Y, (Y / scale).contiguous()   # working set; unit columns: the Gram matrix has a unit diagonal
        self.U = self.X = None                        # factors of the polishing rounds: allocated for the working set only
        self.info = torch.zeros(B, dtype=torch.int32, device=Y.device)
        self.final = None                             # allocated when the first matrix is done
        self.redo = []                                # matrices handed to the library at the end
        self.finished = False
        self.rounds = 0                               # factorisation rounds enqueued so far
        self.repairs = 0                              # matrices swept a second time (see _repair)
        self.repaired_ids = []                        # which matrices of the stack those were
        self.gram = self.far = None
        # The bookkeeping lives on the host (it waits once per round anyway), per working-set entry:
        # which matrix of the stack it is and whether it is within ||G - I||_F < 0.5.
        self.ids = np.arange(B)
        self.near = np.zeros(B, dtype=bool)
        self.last = None                              # (pivot flags, near, ids) of the round not yet looked at
        self.far_before = np.full(B, np.inf)          # per working-set entry: ||G - I||_F^2 at the test before this one if it was far
        self.stuck = np.zeros(B, dtype=np.int64)      # per working-set entry: rounds in a row that did not halve that distance
        self.mended = np.zeros(B, dtype=bool)         # per working-set entry: has been through the replacing sweep
        self.stale = False                            # the Gram matrices are those of before a repair: no round on them
        self.swept = sweep
        if sweep:
            # One sweep of block Gram-Schmidt with reorthogonalisation.  Where no pivot of a panel factorisation
            # came near the floor and no column had to be replaced (info == 0) the result is orthonormal to
            # fp32 rounding by construction; the rounds below are for the other matrices only.
            # replace_first: the caller knows the stack to be of low numerical rank (its last update needed the
            # replacing sweep for most matrices) and goes there directly
            block_gram_schmidt(self.Q, self.info, pivot_floor, replace_dependent=replace_first, true_n=self.true_n)
            if replace_first:
                self.mended[:] = True
            self.info_host = self._to_host(self.info)

    def _to_host(self, t):
        """A copy of a small device tensor on its way into pinned host memory, queued on the current stream right
        behind what produced it (read it with _landed_numpy).  The host never queues a copy at the moment it wants
        the data: on a stream that shares a hardware queue with another stack's chain of launches such a copy, and the
        host with it, would wait for that whole chain."""
        host = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
        host.copy_(t, non_blocking=True)
        landed = torch.cuda.Event()
        landed.record(torch.cuda.current_stream(self.device))
        return host, landed

    @staticmethod
    def _landed_numpy(pair):
        host, landed = pair
        landed.synchronize()
        return host.numpy()

    def _padded(self, Y):
        """Orders that are not a multiple of 64: diag(Y, I)."""
        padded = torch.zeros(Y.shape[0], self.n, self.n, device=Y.device)
        padded[:, :self.true_n, :self.true_n] = Y
        padded.diagonal(dim1=1, dim2=2)[:, self.true_n:] = 1.0
        return padded

    def _original(self, ids):
        """The matrices `ids` (int64 GPU vector) of the stack the object was made for."""
        if self.Y is not None:
            return self.Y.index_select(0, ids)
        again = self.remake(ids)
        return self._padded(again) if self.n != self.true_n else again

    def _index(self, positions):
        # (through pinned memory and without waiting: see _to_host)
        host = torch.as_tensor(np.ascontiguousarray(positions), dtype=torch.int64).pin_memory()
        return host.to(self.Q.device, non_blocking=True)

    def _finish(self, where, source):
        """The working-set entries `where` (host positions) of `source` are final."""
        if where.size == 0:
            return
        B = self.batch
        if self.final is None and where.size == B and source.shape[0] == B and np.array_equal(self.ids, np.arange(B)):
            self.final = source                       # the whole stack at once: no copy
            return
        if self.final is None:
            self.final = torch.empty(B, self.n, self.n, device=self.device)
        self.final.index_copy_(0, self._index(self.ids[where]), source.index_select(0, self._index(where)))

    def _keep(self, keep):
        """Shrink the working set to the entries of the host mask `keep`."""
        if keep.all():
            return
        index = self._index(np.nonzero(keep)[0])
        self.Q = self.Q.index_select(0, index)
        if self.gram is not None:
            self.gram = self.gram.index_select(0, index)
        self.ids, self.near, self.mended = self.ids[keep], self.near[keep], self.mended[keep]
        self.far_before, self.stuck = self.far_before[keep], self.stuck[keep]

    def check(self):
        if self.swept:
            self.swept = False
            clean = self._landed_numpy(self.info_host) == 0                     # (waits for the sweep, if it is not through)
            clean[self.leave] = True
            # the clean matrices are final where they are; only the flagged ones are copied out into a working
            # set of their own and written back when they are done
            self.final = self.Q
            self._keep(~clean)
            self.finished = self.ids.size == 0
            if self.finished:
                return
        self.gram = gemm(self.Q, self.Q, trans_a=True, symmetric=True)
        self.far = gram_deviation(self.gram)                                    # max |G - I|, ||G - I||_F^2
        self.far_host = self._to_host(self.far)

    def _repair(self, where):
        """The working-set entries `where` (host positions) are far from orthonormal after the sweep: matrices of low
        numerical rank, where what a first pass leaves of a dependent column is rounding noise and a second pass
        cannot mend it (columns end unnormalised or parallel, and Cholesky QR rounds on such a matrix diverge).  They
        are swept again from their original columns, three passes, with every column that a pass finds dependent
        replaced by a stand-in column (block_gram_schmidt(replace_dependent=True))."""
        original = self._original(self._index(self.ids[where]))
        scale = torch.linalg.vector_norm(original, dim=1, keepdim=True).clamp_min(1e-30)
        again = (original / scale).contiguous()
        info = torch.zeros(again.shape[0], dtype=torch.int32, device=again.device)
        block_gram_schmidt(again, info, self.pivot_floor, replace_dependent=True, true_n=self.true_n)
        self.Q.index_copy_(0, self._index(where), again)
        self.repairs += int(where.size)
        self.repaired_ids += [int(i) for i in self.ids[where]]

    def _failures(self):
        """Host mask over the entries of the last round: the factorisation met a NaN."""
        info, near, ids = self.last
        self.last = None
        return (self._landed_numpy(info)[:ids.size] & 1) != 0, near, ids

    def poll(self):
        if self.finished:
            return True
        far = self._landed_numpy(self.far_host)                                 # the host synchronisation
        failed = np.zeros(self.ids.size, dtype=bool)
        if self.last is not None:
            bad, near, ids = self._failures()
            self.redo += ids[bad & near].tolist()                               # (already finalised, wrongly)
            failed |= bad[~near]                                                # the entries still in the working set
        with np.errstate(invalid="ignore"):
            done = far[:, 0] < self.tolerance                                   # False for NaN as well
            self.near = far[:, 1] < 0.25
        if self.rounds_left == 0:
            failed |= ~done
        done &= ~failed
        self.redo += self.ids[failed].tolist()
        self._finish(np.nonzero(done)[0], self.Q)
        distance = far[:, 1][~(done | failed)]
        self._keep(~(done | failed))
        self.finished = self.ids.size == 0
        if not self.finished:
            # A matrix that is far from orthonormal after the sweep usually has a few stand-in columns that are a
            # little off, and a round or two mend it (a round may first throw it further off).  One that two rounds
            # in a row did not bring nearer than half of before -- or a stack where every fourth matrix is far (eight
            # at least) -- is of low numerical rank: rounds diverge there, the replacing sweep does not.
            away = ~self.near
            many = away.sum() >= 8 and away.sum() * 4 > self.batch
            with np.errstate(invalid="ignore"):
                no_nearer = away & np.isfinite(self.far_before) & ~(distance < 0.5 * self.far_before)      # (NaN and inf count)
            self.stuck = np.where(no_nearer, self.stuck + 1, 0)
            again = away & ~self.mended & ((self.stuck >= 2) | many)
            if again.any():
                self._repair(np.nonzero(again)[0])
                self.mended |= again
                self.stale = True
                self.rounds_left = min(self.rounds_left, 3)   # what is far after the repair and three rounds goes to the library
            self.far_before = np.where(away, distance, np.inf)
        return self.finished

    def advance(self):
        if self.stale:                                # repaired matrices are tested first (the next check())
            self.stale, self.gram = False, None
            return
        k = self.ids.size
        info = self.info[:k]
        info.zero_()
        if self.U is None:
            self.U = torch.empty_like(self.Q)
            self.X = torch.zeros_like(self.Q)         # inverse factors; the part below the diagonal blocks stays zero
        cholesky_upper(self.gram, self.U[:k], self.X[:k], info, self.pivot_floor)
        out = torch.empty_like(self.Q)
        solve_upper_right(self.Q, self.U[:k], self.X[:k], self.gram, out)      # the Gram matrix is used up: scratch
        self.Q, self.gram = out, None
        self.last = (self._to_host(info), self.near.copy(), self.ids.copy())
        self.rounds_left -= 1
        self.rounds += 1
        if self.near.any():
            # ||G - I||_F < 0.5 before the round: G was positive definite with eigenvalues in (0.5, 1.5),
            # no pivot came near the floor and the round leaves Q orthonormal to rounding
            self._finish(np.nonzero(self.near)[0], self.Q)
            self._keep(~self.near)
            self.finished = self.ids.size == 0

    def result(self):
        if self.last is not None:                     # pivot flags of the last round
            bad, near, ids = self._failures()
            self.redo += ids[bad & near].tolist()
        if self.final is None:
            self.final = torch.empty(self.batch, self.n, self.n, device=self.device)
        if self.redo:
            redo = torch.tensor(sorted(set(self.redo)), device=self.device)
            torch.cuda.synchronize()              # the library routine is not trusted to be stream-ordered here
            self.final[redo] = _householder_qr(self._original(redo))[0]
            torch.cuda.synchronize()
        Q = self.final
        if Q.shape[1] != self.true_n:
            Q = Q[:, :self.true_n, :self.true_n].contiguous()
        return Q, len(set(self.redo))


def cholesky_qr(Y, max_rounds=12, pivot_floor=PIVOT_FLOOR, tolerance=2e-5):
    """(Q, number of matrices redone by the library) for one stack; see CholeskyQR."""
    state = CholeskyQR(Y, max_rounds, pivot_floor, tolerance)
    while not state.finished:
        state.check()
        if not state.poll():
            state.advance()
    return state.result()
