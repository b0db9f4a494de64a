"""TEST INFRASTRUCTURE, NOT PRODUCT CODE -- numpy / pure-Python restatements of the
reference's CPU blockwise quantizer, plus the ctypes binding of oracle/qoracle.c.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.

Reference lines restated (relative to the reference checkout):
  qtensor/functional.py:87-113    code-map builders      -> dynamic_map / linear_map
  qtensor/functional.py:526-615   _quantize_blockwise_cpu   -> quantize_np / quantize_py
  qtensor/functional.py:618-688   _dequantize_blockwise_cpu -> dequantize_np / dequantize_py
  qtensor/functional.py:703-715   _nearest_code_indices     -> _nearest_np / _nearest_py
  qtensor/functional.py:718-746   _pack_indices / _unpack_indices -> pack_np / unpack_np

Three independent forms exist on purpose (C scalar, numpy whole-array, Python scalar
with exact rational checks in the tests); they are pinned against each other and
against known-answer vectors in tests/test_oracle_quant.py.

Parity notes:
  * code-map *bits* are not fixed by the written algorithm: the reference builds them
    with torch.linspace, whose float32 CPU kernel depends on the host's vector width.
    linear_map / dynamic_map below are the closed forms in float64 rounded once to
    float32 and agree with the reference to 1 ulp; bit-exact maps come from
    tests/golden/reference_vectors.npz.  Code maps are an *input* of the quantizer.
  * a code table with repeated entries that is also unsorted: parity unpinned (sort
    order among equal keys is unspecified in the reference); neither shipped map has
    repeated entries.
"""
from __future__ import annotations

import ctypes as ct
import subprocess
from fractions import Fraction
from pathlib import Path

import numpy as np

F32 = np.float32
_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "libqoracle.so"
_lib = None


# --------------------------------------------------------------------------- code maps
def linear_map(signed: bool = True, total_bits: int = 8, power: int = 2) -> np.ndarray:
    """functional.py:106-113 in closed form (float64, one rounding to float32)."""
    n = 2 ** total_bits
    if signed:
        data = np.linspace(-1.0, 1.0, n, dtype=np.float64)
        data[2 ** (total_bits - 1) - 1] = 0.0
    else:
        data = np.linspace(0.0, 1.0, n, dtype=np.float64)
    data = data.astype(F32).astype(np.float64)          # the reference holds float32 here
    return (np.sign(data) * np.abs(data) ** power).astype(F32)


def dynamic_map(signed: bool = True, total_bits: int = 8, power: int = 1) -> np.ndarray:
    """functional.py:87-103: for each of the total_bits-1 exponent levels i, the
    midpoints of 2**i (signed) equal cells of [0.1, 1], scaled by 10**(i-(bits-2)),
    mirrored when signed, plus the two entries 0 and 1."""
    levels = total_bits - 1
    vals: list[float] = []
    for i in range(levels):
        cells = 2 ** i + 1 if signed else 2 ** (i + 1) + 1
        edges = np.linspace(0.1, 1.0, cells, dtype=np.float64).astype(F32)
        mids = ((edges[:-1] + edges[1:]) / F32(2.0)).astype(F32)
        scale = 10.0 ** (-(levels - 1) + i)
        vals += [scale * float(m) for m in mids]
        if signed:
            vals += [-scale * float(m) for m in mids]
    vals += [0.0, 1.0]
    vals.sort()
    data = np.asarray(vals, dtype=np.float64).astype(F32).astype(np.float64)
    return (np.sign(data) * np.abs(data) ** power).astype(F32)


# --------------------------------------------------------------------------- bf16
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bfloat16, returned as uint16 bit patterns; every NaN
    becomes 0x7FC0 like torch's CPU cast."""
    u = np.ascontiguousarray(x, dtype=F32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, 0x7FC0, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(F32)


# --------------------------------------------------------------------------- packing
def pack_np(idx: np.ndarray, bits: int) -> np.ndarray:
    """Flat index stream -> bytes; 4-bit puts the FIRST element in the HIGH nibble and
    pads an odd tail with a zero nibble."""
    idx = np.asarray(idx).astype(np.uint8).reshape(-1)
    if bits == 8:
        return idx.copy()
    if idx.size % 2:
        idx = np.concatenate([idx, np.zeros(1, np.uint8)])
    pairs = idx.reshape(-1, 2)
    return ((pairs[:, 0] << 4) + (pairs[:, 1] & 15)).astype(np.uint8)


def unpack_np(packed: np.ndarray, numel: int, bits: int) -> np.ndarray:
    packed = np.asarray(packed, dtype=np.uint8).reshape(-1)
    if bits == 8:
        return packed[:numel].astype(np.int64)
    both = np.stack([packed >> 4, packed & 15], axis=1).reshape(-1)
    return both[:numel].astype(np.int64)


# --------------------------------------------------------------------------- numpy form
def _sorted_code(code: np.ndarray):
    code = np.asarray(code, dtype=F32).reshape(-1)
    if np.any(code[1:] < code[:-1]):
        perm = np.argsort(code, kind="stable")
        return code[perm], perm
    return code, None


def _nearest_np(v: np.ndarray, code_sorted: np.ndarray) -> np.ndarray:
    n = code_sorted.size
    ins = np.searchsorted(code_sorted, v, side="right")        # NaN sorts last -> n
    lo = np.clip(ins - 1, 0, None)
    hi = np.clip(ins, None, n - 1)
    with np.errstate(invalid="ignore"):
        dlo = np.abs((v - code_sorted[lo]).astype(F32))
        dhi = np.abs((code_sorted[hi] - v).astype(F32))
        return np.where(dlo > dhi, hi, lo)


def quantize_np(A, code, order: int, blocksize: int, bits: int, store_diag: bool = False):
    """Whole-array restatement.  A: float32 array with order*order entries.
    Returns (out uint8, absmax float32[, diag float32])."""
    if bits not in (4, 8):
        raise ValueError(f"unsupported bit width {bits}")
    if blocksize <= 0:
        raise ValueError("blocksize must be positive")
    work = np.array(A, dtype=F32).reshape(order, order)
    code_sorted, perm = _sorted_code(code)
    if code_sorted.size != 2 ** bits:
        raise ValueError("code table must hold 2**bits entries")
    diag = None
    if store_diag:
        diag = work.diagonal().copy()
        work[np.arange(order), np.arange(order)] = 0.0
    nb = -(-order // blocksize)
    padded = np.zeros((order, nb * blocksize), dtype=F32)
    padded[:, :order] = work
    seg = padded.reshape(order, nb, blocksize)
    mag = np.abs(seg)
    amax = mag.max(axis=2)                                      # np.max propagates NaN
    amax = np.where(np.isnan(amax), F32(np.nan), amax).astype(F32)
    with np.errstate(divide="ignore", invalid="ignore"):
        v = (seg / amax[:, :, None]).astype(F32)
        # clip keeps NaN as NaN, like torch.clamp
        v = np.where(np.isnan(v), v, np.clip(v, code_sorted[0], code_sorted[-1])).astype(F32)
    idx = _nearest_np(v, code_sorted)
    if perm is not None:
        idx = perm[idx]
    idx = np.where((amax == 0)[:, :, None], 0, idx)
    idx = idx.reshape(order, nb * blocksize)[:, :order].reshape(-1)
    out = pack_np(idx, bits)
    absmax = amax.reshape(-1).astype(F32)
    if store_diag:
        return out, absmax, diag.astype(F32)
    return out, absmax


def dequantize_np(q, code, order: int, absmax, blocksize: int, bits: int, diag=None,
                  to_bf16: bool = False) -> np.ndarray:
    """Returns float32 [order, order]; with to_bf16 the values are rounded to bfloat16
    (still stored as float32) so they can be compared with a bf16 device result."""
    if bits not in (4, 8):
        raise ValueError(f"unsupported bit width {bits}")
    nb = -(-order // blocksize)
    absmax = np.asarray(absmax, dtype=F32).reshape(-1)
    if absmax.size != order * nb:
        raise ValueError(f"absmax has {absmax.size} entries, expected {order * nb}")
    code = np.asarray(code, dtype=F32).reshape(-1)
    idx = unpack_np(q, order * order, bits).reshape(order, order)
    scale = np.repeat(absmax.reshape(order, nb), blocksize, axis=1)[:, :order]
    with np.errstate(invalid="ignore", over="ignore"):
        vals = (code[idx] * scale).astype(F32)
    vals = np.where(scale == 0, F32(0.0), vals).astype(F32)
    if to_bf16:
        vals = bf16_bits_to_f32(f32_to_bf16_bits(vals)).reshape(order, order)
    if diag is not None:
        d = np.asarray(diag, dtype=F32).reshape(-1)
        if d.size != order:
            raise ValueError(f"diag must have length {order}")
        if to_bf16:
            d = bf16_bits_to_f32(f32_to_bf16_bits(d))
        vals = vals.copy()
        vals[np.arange(order), np.arange(order)] = d
    return vals


# --------------------------------------------------------------------------- scalar form
def _nearest_py(v: F32, code_sorted: np.ndarray) -> int:
    n = len(code_sorted)
    if np.isnan(v):
        ins = n
    else:
        ins = sum(1 for c in code_sorted if c <= v)
    lo = max(ins - 1, 0)
    hi = min(ins, n - 1)
    dlo = abs(F32(v - code_sorted[lo]))
    dhi = abs(F32(code_sorted[hi] - v))
    return hi if dlo > dhi else lo


def quantize_py(A, code, order: int, blocksize: int, bits: int, store_diag: bool = False):
    """Element-at-a-time Python loops; for tiny inputs only."""
    work = np.array(A, dtype=F32).reshape(order, order)
    code_sorted, perm = _sorted_code(code)
    nb = -(-order // blocksize)
    absmax = np.zeros(order * nb, dtype=F32)
    diag = np.zeros(order, dtype=F32)
    idx = np.zeros(order * order, dtype=np.int64)
    with np.errstate(divide="ignore", invalid="ignore"):
        for r in range(order):
            if store_diag:
                diag[r] = work[r, r]
                work[r, r] = 0.0
            for b in range(nb):
                c0, c1 = b * blocksize, min((b + 1) * blocksize, order)
                amax = F32(0.0)
                for c in range(c0, c1):
                    a = abs(work[r, c])
                    if np.isnan(a) or np.isnan(amax):
                        amax = F32(np.nan)
                    elif a > amax:
                        amax = a
                absmax[r * nb + b] = amax
                if amax == 0:
                    continue
                for c in range(c0, c1):
                    v = F32(work[r, c] / amax)
                    if not np.isnan(v):
                        v = min(max(v, code_sorted[0]), code_sorted[-1])
                    k = _nearest_py(v, code_sorted)
                    idx[r * order + c] = k if perm is None else perm[k]
    out = pack_np(idx, bits)
    if store_diag:
        return out, absmax, diag
    return out, absmax


def nearest_exact(v: float, code_sorted) -> tuple[int, bool]:
    """Index of the table entry nearest to v in exact rational arithmetic (lower index on
    an exact tie) and whether v lies exactly midway between its two neighbours."""
    fv = Fraction(float(v))
    best, best_d, tie = 0, None, False
    for i, c in enumerate(code_sorted):
        d = abs(fv - Fraction(float(c)))
        if best_d is None or d < best_d:
            best, best_d, tie = i, d, False
        elif d == best_d:
            tie = True
    return best, tie


# --------------------------------------------------------------------------- C binding
def build_c_oracle(force: bool = False) -> Path:
    src = _HERE / "qoracle.c"
    if force or not _LIB_PATH.is_file() or _LIB_PATH.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-C", str(_HERE), "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def c_lib() -> ct.CDLL:
    global _lib
    if _lib is None:
        build_c_oracle()
        _lib = ct.CDLL(str(_LIB_PATH))
        _lib.qo_quantize.restype = ct.c_int
        _lib.qo_dequantize.restype = ct.c_int
        _lib.qo_quantize.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_int,
                                     ct.c_int, ct.c_void_p, ct.c_void_p, ct.c_void_p]
        _lib.qo_dequantize.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_int, ct.c_int, ct.c_int,
                                       ct.c_void_p, ct.c_void_p, ct.c_void_p]
    return _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ct.c_void_p)


def quantize_c(A, code, order: int, blocksize: int, bits: int, store_diag: bool = False):
    A = np.ascontiguousarray(A, dtype=F32).reshape(-1)
    if A.size != order * order:
        raise ValueError(f"expected {order * order} elements, found {A.size}")
    code = np.ascontiguousarray(code, dtype=F32).reshape(-1)
    if code.size != 2 ** bits:
        raise ValueError("code table must hold 2**bits entries")
    nb = -(-order // blocksize)
    absmax = np.empty(order * nb, dtype=F32)
    diag = np.empty(max(order, 1), dtype=F32)
    out = np.empty((order * order * bits + 7) // 8, dtype=np.uint8)
    rc = c_lib().qo_quantize(_ptr(A), _ptr(code), order, blocksize, bits, int(store_diag),
                             _ptr(absmax), _ptr(diag), _ptr(out))
    if rc:
        raise RuntimeError(f"qo_quantize failed with code {rc}")
    if store_diag:
        return out, absmax, diag[:order]
    return out, absmax


def dequantize_c(q, code, order: int, absmax, blocksize: int, bits: int, diag=None,
                 to_bf16: bool = False) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.uint8).reshape(-1)
    code = np.ascontiguousarray(code, dtype=F32).reshape(-1)
    absmax = np.ascontiguousarray(absmax, dtype=F32).reshape(-1)
    nb = -(-order // blocksize)
    if absmax.size != order * nb:
        raise ValueError(f"absmax has {absmax.size} entries, expected {order * nb}")
    d = None if diag is None else np.ascontiguousarray(diag, dtype=F32).reshape(-1)
    if to_bf16 and d is not None:
        d = bf16_bits_to_f32(f32_to_bf16_bits(d))
    out = np.empty(order * order, dtype=F32)
    rc = c_lib().qo_dequantize(_ptr(q), _ptr(code), order, blocksize, bits, _ptr(absmax),
                               None if d is None else _ptr(d), _ptr(out))
    if rc:
        raise RuntimeError(f"qo_dequantize failed with code {rc}")
    if to_bf16:
        out = out.reshape(order, order)
        dsave = out.diagonal().copy() if d is not None else None
        out = bf16_bits_to_f32(f32_to_bf16_bits(out.reshape(-1))).reshape(order, order).copy()
        if dsave is not None:
            out[np.arange(order), np.arange(order)] = dsave
        return out
    return out.reshape(order, order)
