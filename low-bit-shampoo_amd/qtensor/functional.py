"""Blockwise 4/8-bit quantization of square matrices on MI355X.

Public surface and argument meaning follow the reference's qtensor/functional.py
(quantize_blockwise :116-178, dequantize_blockwise :181-236, quantize_blockwise_diagreal
:239-309, dequantize_blockwise_diagreal :312-368, code-map builders :87-113, get_ptr
:68-84, compute_power :749-762, module globals lib / lib_quan / lib_dequan /
lib_quan_diagreal / lib_dequan_diagreal :12-65).  Every tensor that reaches these functions
must live on the GPU: the work is done by libqtensor_hip.so (hand-written gfx950 kernels)
through ctypes, with the arithmetic of the reference's CPU path (true fp32 division by the
segment maximum, ties to the lower index, first element of a pair in the high nibble).

Deliberate differences from the reference:
  * there is no CPU or MPS fallback here: a tensor that is not on the GPU, or a missing
    library, raises instead of computing somewhere else;
  * dequantize_blockwise_diagreal returns its result (the reference falls off the end of
    the function and returns None, :312-368);
  * launches go to torch's current stream of the tensor's device instead of the null stream;
  * argument shapes are validated before the launch and native errors raise RuntimeError.
"""
import ctypes as ct
from typing import Optional, Tuple

import torch
from torch import Tensor

from qtensor.cextension import get_lib

try:
    lib = get_lib()
except Exception:  # same policy as the reference: import never fails, use does
    lib = None

_BLOCKSIZES = (2048, 1024, 512, 256, 128, 64)
_MISSING = ("HIP quantization library is unavailable; build low-bit-shampoo_amd/csrc "
            "(csrc/build.sh) on a ROCm build of PyTorch.")

if lib is not None:
    lib_quan = {
        8: (lib.cquantize_blockwise_8bit_fp32, lib.cquantize_blockwise_8bit_bf16),
        4: (lib.cquantize_blockwise_4bit_fp32, lib.cquantize_blockwise_4bit_bf16),
    }
    lib_dequan = {
        8: (lib.cdequantize_blockwise_8bit_fp32, lib.cdequantize_blockwise_8bit_bf16),
        4: (lib.cdequantize_blockwise_4bit_fp32, lib.cdequantize_blockwise_4bit_bf16),
    }
    lib_quan_diagreal = {
        8: (lib.cquantize_blockwise_diagreal_8bit_fp32, lib.cquantize_blockwise_diagreal_8bit_bf16),
        4: (lib.cquantize_blockwise_diagreal_4bit_fp32, lib.cquantize_blockwise_diagreal_4bit_bf16),
    }
    lib_dequan_diagreal = {
        8: (lib.cdequantize_blockwise_diagreal_8bit_fp32, lib.cdequantize_blockwise_diagreal_8bit_bf16),
        4: (lib.cdequantize_blockwise_diagreal_4bit_fp32, lib.cdequantize_blockwise_diagreal_4bit_bf16),
    }

    def _bind_stream_variants():
        P, I = ct.c_void_p, ct.c_int
        table = {}
        for bits in (8, 4):
            for di, dt in enumerate(("fp32", "bf16")):
                for diag in (False, True):
                    mid = "_diagreal" if diag else ""
                    for kind in ("quantize", "dequantize"):
                        fn = getattr(lib, f"c{kind}_blockwise{mid}_{bits}bit_{dt}_stream")
                        fn.restype = None
                        fn.argtypes = [P, P, I, P] + ([P] if diag else []) + [P, I, P]
                        table[(kind, bits, di, diag)] = fn
        lib.qtensor_hip_last_error.restype = ct.c_int
        lib.qtensor_hip_last_error_string.restype = ct.c_char_p
        return table

    _STREAM_FN = _bind_stream_variants()
else:
    lib_quan = {}
    lib_dequan = {}
    lib_quan_diagreal = {}
    lib_dequan_diagreal = {}
    _STREAM_FN = {}


def get_ptr(A: Optional[Tensor]) -> Optional[ct.c_void_p]:
    """ctypes pointer to a tensor's storage, None for None (reference :68-84)."""
    return None if A is None else ct.c_void_p(A.data.data_ptr())


# ----------------------------------------------------------------------------- code maps
def create_dynamic_map(signed=True, total_bits=8, power=1):
    """"Dynamic tree" table: total_bits-1 exponent levels; level i holds the midpoints of
    2**i (signed) or 2**(i+1) (unsigned) equal cells of [0.1, 1] scaled by
    10**(i - (total_bits-2)); both signs when signed; plus 0 and 1 (reference :87-103)."""
    levels = total_bits - 1
    entries = []
    for i in range(levels):
        cells = 2 ** i + 1 if signed else 2 ** (i + 1) + 1
        edges = torch.linspace(0.1, 1, cells)
        mids = (edges[:-1] + edges[1:]) / 2.0
        scale = 10 ** (-(levels - 1) + i)
        entries += (scale * mids).tolist()
        if signed:
            entries += (-scale * mids).tolist()
    entries += [0, 1.0]
    entries.sort()
    table = torch.Tensor(entries)
    return table.sign() * table.abs().pow(power)


def create_linear_map(signed=True, total_bits=8, power=2):
    """Evenly spaced grid on [-1, 1] (or [0, 1]) pushed through sign(x)|x|**power; the signed
    grid has its entry just below the middle forced to exactly 0 (reference :106-113)."""
    count = 2 ** total_bits
    if signed:
        grid = torch.linspace(-1, 1, count)
        grid[count // 2 - 1] = 0
    else:
        grid = torch.linspace(0, 1, count)
    return grid.sign() * grid.abs().pow(power)


# ----------------------------------------------------------------------------- helpers
def _absmax_len(order: int, blocksize: int) -> int:
    return order * (-(-order // blocksize))


def _packed_len(order: int, bits: int) -> int:
    per_byte = 8 // bits
    return -(-(order * order) // per_byte)


def _require_gpu(A: Tensor, what: str) -> None:
    if not A.is_cuda:
        raise RuntimeError(
            f"{what}: tensor is on '{A.device}'. This build computes on the GPU only and has no "
            "CPU or MPS fallback; move the tensor to the GPU.")
    if lib is None:
        raise RuntimeError(_MISSING)


def _dtype_slot(dtype: torch.dtype, what: str) -> int:
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise ValueError(f"data type of {what} is not supported: {dtype}")


def _check_buffer(t: Tensor, name: str, numel: int, dtype: torch.dtype, device: torch.device) -> None:
    if t.device != device:
        raise ValueError(f"{name} tensor must live on the same device as the data ({t.device} vs {device}).")
    if t.dtype != dtype:
        raise ValueError(f"{name} has dtype {t.dtype}, expected {dtype}.")
    if t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} entries, expected {numel}.")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous.")


def _check_common(code: Tensor, order: int, blocksize: int, bits: int, device: torch.device) -> None:
    assert blocksize in _BLOCKSIZES
    assert code.shape == torch.Size([2 ** bits])
    if bits not in (4, 8):
        raise ValueError(f"Unsupported bit width: {bits}")
    if order < 1 or order * order >= 2 ** 31:
        raise ValueError(f"order {order} out of range: need 1 <= order and order*order < 2**31.")
    _check_buffer(code, "code", 2 ** bits, torch.float32, device)


def _call(fn, device: torch.device, *args) -> None:
    stream = torch.cuda.current_stream(device).cuda_stream
    if device.index is not None and device.index != torch.cuda.current_device():
        with torch.cuda.device(device):
            fn(*args, stream)
    else:
        fn(*args, stream)
    if lib.qtensor_hip_last_error():
        raise RuntimeError("libqtensor_hip: " + lib.qtensor_hip_last_error_string().decode())


def _quantize(A, code, order, absmax, diag, out, blocksize, bits, with_diag):
    _require_gpu(A, "quantize_blockwise")
    slot = _dtype_slot(A.dtype, "A")
    _check_common(code, order, blocksize, bits, A.device)
    if A.numel() != order * order:
        raise ValueError(f"Expected tensor with {order * order} elements, found {A.numel()}.")
    if not A.is_contiguous():
        raise ValueError("A must be contiguous.")
    if absmax is None:
        absmax = torch.empty((_absmax_len(order, blocksize),), device=A.device, dtype=torch.float32)
    else:
        _check_buffer(absmax, "absmax", _absmax_len(order, blocksize), torch.float32, A.device)
    if with_diag:
        if diag is None:
            diag = torch.empty((order,), device=A.device, dtype=torch.float32)
        else:
            _check_buffer(diag, "diag", order, torch.float32, A.device)
    if out is None:
        out = torch.empty(_packed_len(order, bits), device=A.device, dtype=torch.uint8)
    else:
        _check_buffer(out, "out", _packed_len(order, bits), torch.uint8, A.device)
    fn = _STREAM_FN[("quantize", bits, slot, with_diag)]
    if with_diag:
        _call(fn, A.device, A.data_ptr(), code.data_ptr(), order, absmax.data_ptr(), diag.data_ptr(),
              out.data_ptr(), blocksize)
    else:
        _call(fn, A.device, A.data_ptr(), code.data_ptr(), order, absmax.data_ptr(), out.data_ptr(), blocksize)
    return out, absmax, diag


def _dequantize(A, code, order, absmax, diag, outdtype, out, blocksize, bits, with_diag):
    _require_gpu(A, "dequantize_blockwise")
    if out is None:
        out = torch.empty((order, order), device=A.device, dtype=outdtype)
    slot = _dtype_slot(out.dtype, "out")
    _check_common(code, order, blocksize, bits, A.device)
    _check_buffer(A, "A", _packed_len(order, bits), torch.uint8, A.device)
    _check_buffer(absmax, "absmax", _absmax_len(order, blocksize), torch.float32, A.device)
    _check_buffer(out, "out", order * order, out.dtype, A.device)
    if with_diag:
        _check_buffer(diag, "diag", order, torch.float32, A.device)
    fn = _STREAM_FN[("dequantize", bits, slot, with_diag)]
    if with_diag:
        _call(fn, A.device, A.data_ptr(), code.data_ptr(), order, absmax.data_ptr(), diag.data_ptr(),
              out.data_ptr(), blocksize)
    else:
        _call(fn, A.device, A.data_ptr(), code.data_ptr(), order, absmax.data_ptr(), out.data_ptr(), blocksize)
    return out


# ----------------------------------------------------------------------------- public API
def quantize_blockwise(
    A: Tensor,
    code: Tensor,
    order: int,
    absmax: Optional[Tensor] = None,
    out: Optional[Tensor] = None,
    blocksize: int = 256,
    bits: int = 8,
) -> Tuple[Tensor, Tensor]:
    """Quantize the order x order matrix A (fp32 or bf16, contiguous) against `code`.

    Returns (out, absmax): out uint8[ceil(order*order*bits/8)], absmax
    fp32[order*ceil(order/blocksize)].  Passed-in buffers are reused."""
    out, absmax, _ = _quantize(A, code, order, absmax, None, out, blocksize, bits, False)
    return out, absmax


def dequantize_blockwise(
    A: Tensor,
    code: Tensor,
    order: int,
    absmax: Tensor,
    outdtype=torch.float32,
    out: Optional[Tensor] = None,
    blocksize: int = 256,
    bits: int = 8,
) -> Tensor:
    """Inverse of quantize_blockwise; returns an order x order tensor of `outdtype`
    (fp32 or bf16), or fills and returns `out`."""
    return _dequantize(A, code, order, absmax, None, outdtype, out, blocksize, bits, False)


def quantize_blockwise_diagreal(
    A: Tensor,
    code: Tensor,
    order: int,
    absmax: Optional[Tensor] = None,
    diag: Optional[Tensor] = None,
    out: Optional[Tensor] = None,
    blocksize: int = 256,
    bits: int = 8,
) -> Tuple[Tensor, Tensor, Tensor]:
    """As quantize_blockwise, but the diagonal is kept exactly in diag (fp32[order]) and
    counts as zero for the segment maxima and the codes.  Returns (out, absmax, diag)."""
    return _quantize(A, code, order, absmax, diag, out, blocksize, bits, True)


def dequantize_blockwise_diagreal(
    A: Tensor,
    code: Tensor,
    order: int,
    absmax: Tensor,
    diag: Tensor,
    outdtype=torch.float32,
    out: Optional[Tensor] = None,
    blocksize: int = 256,
    bits: int = 8,
) -> Tensor:
    """Inverse of quantize_blockwise_diagreal: dequantize, then put diag on the diagonal."""
    return _dequantize(A, code, order, absmax, diag, outdtype, out, blocksize, bits, True)


@torch.no_grad()
def compute_power(Vt, S, p, iter_count=4, ridge_epsilon=1e-6, indices=None, max_eigen=None):
    """V^T diag((S + rho)^(-1/p)) V for the kept rows V = Vt[indices], after iter_count
    Bjorck orthonormalisation steps V <- 1.5 V - 0.5 V V^T V; rho = ridge_epsilon times
    max_eigen (or max S) (reference :749-762)."""
    V = Vt if indices is None else Vt[indices]
    top = S.max() if max_eigen is None else max_eigen
    weights = 1 / (S + ridge_epsilon * top).pow(1 / p)
    from qtensor import fused as X
    if X.on_matrix_cores(V) and V.dim() == 2:
        # the same products on the matrix cores (Gram matrices computed as half products and mirrored)
        V = V.contiguous()
        for _ in range(iter_count):
            V = X.gemm(X.gemm(V, V, trans_b=True, symmetric=True), V, addend=V, alpha=-0.5, beta=1.5)
        return X.gemm(V * weights.to(V.dtype).unsqueeze(1), V, trans_a=True, symmetric=True)
    for _ in range(iter_count):
        V = 1.5 * V - 0.5 * V @ V.T @ V
    return V.T @ weights.diag() @ V
