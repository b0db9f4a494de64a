"""Pins for the CPU oracle of the blockwise quantizer (oracle/qoracle.c, quant_np.py,
quant_loop_torch.py).  None of these tests retypes the oracle's formula: they use
known answers, exact rational arithmetic, structural invariants and agreement between
independently written forms."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import quant_np as Q
from oracle import quant_loop_torch as QL

F32 = np.float32
CELLS = [(4, 64), (4, 128), (8, 256), (8, 64), (4, 2048)]


def ulp_distance(a, b):
    ka = a.astype(F32).view(np.int32).astype(np.int64)
    kb = b.astype(F32).view(np.int32).astype(np.int64)
    ka = np.where(ka < 0, -(ka & 0x7FFFFFFF), ka)
    kb = np.where(kb < 0, -(kb & 0x7FFFFFFF), kb)
    return np.abs(ka - kb)


# ------------------------------------------------------------------ code maps
def test_linear_map_known_answer_4bit(code_maps):
    words = ("bf800000 bf4048d2 bf09abce beb851ea be5f0122 bde38e37 bd23d706 00000000 "
             "3b91a2a6 3d23d706 3de38e37 3e5f0122 3eb851ea 3f09abce 3f4048d2 3f800000").split()
    expect = np.array([int(w, 16) for w in words], dtype=np.uint32).view(F32)
    assert np.array_equal(code_maps[("linear-2", 4)].view(np.uint32), expect.view(np.uint32))


@pytest.mark.parametrize("bits", [4, 8])
def test_linear_map_structure_and_closed_form(code_maps, bits):
    m = code_maps[("linear-2", bits)]
    n = 2 ** bits
    assert m.shape == (n,) and m.dtype == F32
    assert np.all(np.diff(m) > 0)
    assert m[0] == -1 and m[-1] == 1 and m[n // 2 - 1] == 0 and not np.signbit(m[n // 2 - 1])
    # antisymmetric except for the slot that was forced to zero
    assert np.all(ulp_distance(m[n // 2 + 1:], -m[:n // 2 - 1][::-1]) <= 1)
    k = np.arange(n, dtype=np.float64)
    closed = -1 + 2 * k / (n - 1)
    closed[n // 2 - 1] = 0
    # linspace carries an absolute error of a few 1e-8 that squaring turns into a large
    # relative error near zero, so compare in the un-squared domain
    root = np.sign(m) * np.sqrt(np.abs(m.astype(np.float64)))
    assert np.allclose(root, closed, rtol=0, atol=4e-7)
    mine = Q.linear_map(True, bits, 2).astype(np.float64)
    assert np.allclose(np.sign(mine) * np.sqrt(np.abs(mine)), closed, rtol=0, atol=4e-7)


@pytest.mark.parametrize("bits", [4, 8])
def test_dynamic_map_structure(code_maps, bits):
    m = code_maps[("dynamic", bits)]
    n = 2 ** bits
    assert m.shape == (n,) and np.all(np.diff(m) > 0)
    assert m[-1] == 1.0 and m.min() > -1.0 and 0.0 in m
    pos = m[m > 0][:-1]
    neg = -m[m < 0][::-1]
    assert np.array_equal(pos, neg)                       # mirrored apart from {0, 1}
    assert np.all(ulp_distance(Q.dynamic_map(True, bits, 1), m) <= 4)
    # top level: midpoints of 2**(bits-2) equal cells of [0.1, 1]
    cells = 2 ** (bits - 2)
    mids = 0.1 + 0.9 * (np.arange(cells) + 0.5) / cells
    assert np.allclose(pos[-cells:], mids, rtol=1e-6)
    assert np.isclose(m[m > 0].min(), 0.55 * 10.0 ** (-(bits - 2)), rtol=1e-6)


# ------------------------------------------------------------------ known answers
@pytest.mark.parametrize("fn", [Q.quantize_c, Q.quantize_np, Q.quantize_py])
def test_exact_codes_map_to_themselves(code_maps, fn):
    code = code_maps[("linear-2", 4)]
    order, bs = 64, 64
    A = np.zeros((order, order), F32)
    for r in range(order):
        A[r, :16] = code * F32(2.0 ** (r - 30))          # power-of-two scale: division exact
        A[r, 16:32] = code[::-1] * F32(2.0 ** (r - 30))
    out, absmax = fn(A, code, order, bs, 4)
    idx = Q.unpack_np(out, order * order, 4).reshape(order, order)
    assert np.array_equal(idx[:, :16], np.tile(np.arange(16), (order, 1)))
    assert np.array_equal(idx[:, 16:32], np.tile(np.arange(16)[::-1], (order, 1)))
    assert np.array_equal(idx[:, 32:], np.full((order, 32), 7))   # exact zeros -> the 0.0 entry
    assert np.array_equal(absmax, (2.0 ** (np.arange(order) - 30)).astype(F32))


def _exact_midpoints(code):
    """(i, v): v is fp32, exactly midway between code[i] and code[i+1], with both
    differences exactly representable, so the compare is an exact tie."""
    found = []
    for i in range(len(code) - 1):
        lo, hi = Fraction(float(code[i])), Fraction(float(code[i + 1]))
        mid = (lo + hi) / 2
        v = F32(float(mid))
        if Fraction(float(v)) != mid:
            continue
        d = mid - lo
        if Fraction(float(F32(float(d)))) == d:
            found.append((i, v))
    return found


@pytest.mark.parametrize("fn", [Q.quantize_c, Q.quantize_np, Q.quantize_py])
@pytest.mark.parametrize("name,bits", [("linear-2", 4), ("linear-2", 8), ("dynamic", 8)])
def test_exact_ties_choose_lower_index(code_maps, fn, name, bits):
    code = code_maps[(name, bits)]
    ties = _exact_midpoints(code)
    assert ties, "no exactly representable midpoint in this table"
    order, bs = 64, 64
    A = np.zeros((order, order), F32)
    A[:, 0] = 1.0                                         # absmax = 1 so v == x
    for j, (_, v) in enumerate(ties[: order - 1]):
        A[0, 1 + j] = v
    out, _ = fn(A, code, order, bs, bits)
    idx = Q.unpack_np(out, order * order, bits).reshape(order, order)
    for j, (i, _) in enumerate(ties[: order - 1]):
        assert idx[0, 1 + j] == i
    # one ulp above the midpoint flips to the upper neighbour
    for j, (_, v) in enumerate(ties[: order - 1]):
        A[0, 1 + j] = np.nextafter(v, F32(2.0), dtype=F32)
    out, _ = fn(A, code, order, bs, bits)
    idx = Q.unpack_np(out, order * order, bits).reshape(order, order)
    for j, (i, _) in enumerate(ties[: order - 1]):
        assert idx[0, 1 + j] == i + 1


@pytest.mark.parametrize("fn", [Q.quantize_c, Q.quantize_np, Q.quantize_py])
def test_extremes_zero_and_nan_segments(code_maps, fn):
    code = code_maps[("linear-2", 4)]
    order, bs = 128, 64
    A = np.full((order, order), 0.25, F32)
    A[0, 3] = 5.0          # positive maximum -> last entry
    A[0, 70] = -7.0        # negative maximum -> entry 0
    A[1, :64] = 0.0        # all-zero segment
    A[1, 5] = -0.0
    A[2, 64:] = 1.0
    A[2, 100] = np.nan     # NaN poisons its segment only
    out, absmax = fn(A, code, order, bs, 4)
    idx = Q.unpack_np(out, order * order, 4).reshape(order, order)
    assert idx[0, 3] == 15 and idx[0, 70] == 0
    assert absmax[0] == 5.0 and absmax[1] == 7.0
    assert np.all(idx[1, :64] == 0) and absmax[2] == 0.0 and not np.signbit(absmax[2])
    assert np.all(idx[2, 64:] == 15) and np.isnan(absmax[5])
    assert np.all(idx[2, :64] == Q.unpack_np(out, order * order, 4).reshape(order, order)[3, :64])
    for deq in (Q.dequantize_c, Q.dequantize_np):
        back = deq(out, code, order, absmax, bs, 4)
        assert np.all(back[1, :64] == 0) and not np.any(np.signbit(back[1, :64]))   # +0.0, not code[0]*0
        assert np.all(np.isnan(back[2, 64:]))
        assert back[0, 3] == 5.0 and back[0, 70] == -7.0


def test_nibble_order_and_odd_order_padding(code_maps):
    code = code_maps[("linear-2", 4)]
    order = 3
    A = np.array([[1.0, -1.0, 0.0], [0.0, 1.0, 1.0], [-1.0, -1.0, 1.0]], F32)
    for fn in (Q.quantize_c, Q.quantize_np, Q.quantize_py):
        out, absmax = fn(A, code, order, 64, 4)
        # flat indices: 15 0 7 | 7 15 15 | 0 0 15  -> F0 77 FF 00 F(0 pad)
        assert out.tolist() == [0xF0, 0x77, 0xFF, 0x00, 0xF0]
        assert absmax.tolist() == [1.0, 1.0, 1.0]
    assert Q.pack_np(np.array([1, 2, 3]), 4).tolist() == [0x12, 0x30]
    assert Q.unpack_np(np.array([0x12, 0x30], np.uint8), 3, 4).tolist() == [1, 2, 3]
    assert Q.pack_np(np.array([200, 3]), 8).tolist() == [200, 3]


@pytest.mark.parametrize("fn", [Q.quantize_c, Q.quantize_np, Q.quantize_py])
def test_diagreal_is_plain_quantizer_on_zeroed_diagonal(code_maps, fn):
    rng = np.random.default_rng(3)
    code = code_maps[("linear-2", 4)]
    order, bs = 96, 64
    A = rng.standard_normal((order, order)).astype(F32)
    A[np.arange(order), np.arange(order)] = 1000.0        # would dominate every absmax
    A[5, :64] = 0.0
    A[5, 5] = 3.0                                         # rest of the segment is zero
    out, absmax, diag = fn(A, code, order, bs, 4, store_diag=True)
    assert np.array_equal(diag, A.diagonal())
    Z = A.copy()
    Z[np.arange(order), np.arange(order)] = 0.0
    out2, absmax2 = fn(Z, code, order, bs, 4)
    assert np.array_equal(out, out2) and np.array_equal(absmax, absmax2)
    assert absmax.max() < 10
    idx = Q.unpack_np(out, order * order, 4).reshape(order, order)
    zero_slot = 7
    d = idx.diagonal()
    assert d[5] == 0 and np.all(np.delete(d, 5) == zero_slot)
    back = Q.dequantize_c(out, code, order, absmax, bs, 4, diag=diag)
    assert np.array_equal(back.diagonal(), A.diagonal())


# ------------------------------------------------------------------ exact-arithmetic brute force
@pytest.mark.parametrize("name,bits", [("linear-2", 4), ("dynamic", 4), ("linear-2", 8), ("dynamic", 8)])
def test_nearest_rule_against_exact_rationals(code_maps, name, bits):
    code = code_maps[(name, bits)]
    rng = np.random.default_rng(bits)
    n = 64 * 64
    vals = rng.uniform(-1, 1, n).astype(F32)
    # crowd some samples around the midpoints, where a wrong rule would show
    mids = ((code[:-1].astype(np.float64) + code[1:]) / 2).astype(F32)
    near = np.concatenate([np.nextafter(mids, F32(2)), np.nextafter(mids, F32(-2)), mids])
    vals[: near.size][: n] = near[: n]
    vals[-1] = 1.0
    A = vals.reshape(64, 64).copy()
    A[:, 0] = 1.0                                         # absmax 1 -> v == x exactly
    out, _ = Q.quantize_c(A, code, 64, 64, bits)
    idx = Q.unpack_np(out, n, bits)
    flat = A.reshape(-1)
    ambiguous = 0
    for k in range(n):
        best, tie = Q.nearest_exact(flat[k], code)
        if idx[k] == best:
            continue
        # a disagreement is only legal where fp32 rounding of the two distances can hide
        # the difference: both candidates adjacent and distances within a few ulps
        v = Fraction(float(flat[k]))
        d_best = abs(v - Fraction(float(code[best])))
        d_got = abs(v - Fraction(float(code[idx[k]])))
        assert abs(int(idx[k]) - best) == 1
        assert d_got - d_best <= Fraction(float(np.spacing(F32(max(d_got, d_best)))))
        if tie:
            assert idx[k] < best or idx[k] == min(idx[k], best)
        ambiguous += 1
    assert ambiguous < n // 50


def test_two_neighbour_rule_equals_first_argmin_over_one_binade(code_maps):
    """Exhaustive over every fp32 in [0.25, 0.5): choosing between the two neighbours of
    the insertion point equals argmin |v - code| over the whole table (first minimum)."""
    code = code_maps[("linear-2", 4)]
    lo = np.array([0.25], F32).view(np.uint32)[0]
    hi = np.array([0.5], F32).view(np.uint32)[0]
    v = np.arange(lo, hi, dtype=np.uint32).view(F32)
    got = Q._nearest_np(v, code)
    ref = np.abs(v[:, None] - code[None, :]).astype(F32).argmin(axis=1)
    assert np.array_equal(got, ref)


# ------------------------------------------------------------------ agreement between forms
def _special_matrix(order, seed):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((order, order)).astype(F32)
    A[rng.random((order, order)) < 0.05] = 0.0
    if order >= 8:
        A[1, :] = 0.0
        A[2, : order // 2] *= F32(1e-41)                  # denormals
        A[3, 0] = np.inf
        A[4, order - 1] = np.nan
        A[5, :] *= F32(1e30)
        A[6, 1] = -0.0
    return A


@pytest.mark.parametrize("order", [1, 2, 3, 17, 64, 100, 129, 200])
@pytest.mark.parametrize("bits,bs", CELLS)
@pytest.mark.parametrize("name", ["linear-2", "dynamic"])
def test_c_numpy_torchloop_agree(code_maps, order, bits, bs, name):
    code = code_maps[(name, bits)]
    A = _special_matrix(order, seed=order * 7 + bits)
    for store_diag in (False, True):
        c = Q.quantize_c(A, code, order, bs, bits, store_diag)
        n = Q.quantize_np(A, code, order, bs, bits, store_diag)
        t = QL.quantize_loop(torch.from_numpy(A), torch.from_numpy(code), order, bs, bits, store_diag)
        for x, y, z in zip(c, n, t):
            assert np.array_equal(x, y, equal_nan=True)
            assert np.array_equal(x, z.numpy(), equal_nan=True)
        diag = c[2] if store_diag else None
        dc = Q.dequantize_c(c[0], code, order, c[1], bs, bits, diag=diag)
        dn = Q.dequantize_np(c[0], code, order, c[1], bs, bits, diag=diag)
        dt = QL.dequantize_loop(torch.from_numpy(c[0]), torch.from_numpy(code), order,
                                torch.from_numpy(c[1]), bs, bits,
                                diag=None if diag is None else torch.from_numpy(diag)).numpy()
        assert np.array_equal(dc.view(np.uint32) | 0, dn.view(np.uint32) | 0) or \
            np.array_equal(dc, dn, equal_nan=True)
        assert np.array_equal(np.signbit(dc), np.signbit(dn))
        assert np.array_equal(dc, dt, equal_nan=True)
        assert np.array_equal(np.signbit(dc), np.signbit(dt))


@pytest.mark.parametrize("order", [5, 16, 33])
def test_python_scalar_form_agrees(code_maps, order):
    for (name, bits), code in code_maps.items():
        A = _special_matrix(order, seed=order)
        for store_diag in (False, True):
            c = Q.quantize_c(A, code, order, 64, bits, store_diag)
            p = Q.quantize_py(A, code, order, 64, bits, store_diag)
            for x, y in zip(c, p):
                assert np.array_equal(x, y, equal_nan=True)


def test_bf16_round_trip_helpers_match_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4096).astype(F32) * F32(10.0) ** rng.integers(-20, 20, 4096),
                        np.array([0.0, -0.0, np.inf, -np.inf, 1.00390625, 1.01171875, np.nan, -np.nan], F32)]).astype(F32)
    mine = Q.f32_to_bf16_bits(x)
    theirs = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    finite = ~np.isnan(x)
    assert np.array_equal(mine[finite], theirs[finite])
    # NaN payloads differ between torch's scalar and vectorised casts; any NaN is a NaN
    assert np.all(np.isnan(Q.bf16_bits_to_f32(mine[~finite]))) and np.all(mine[~finite] == 0x7FC0)
    assert np.array_equal(Q.bf16_bits_to_f32(mine), torch.from_numpy(x).to(torch.bfloat16).float().numpy(), equal_nan=True)
    lib = Q.c_lib()
    lib.qo_f32_to_bf16.restype = np.ctypeslib.ctypes.c_uint16
    lib.qo_f32_to_bf16.argtypes = [np.ctypeslib.ctypes.c_float]
    assert all(lib.qo_f32_to_bf16(float(v)) == int(m) for v, m in zip(x[-520:], mine[-520:]))


def test_bf16_output_rounding(code_maps):
    code = code_maps[("linear-2", 4)]
    A = _special_matrix(64, 1)
    A[3, 0] = 1.0
    A[4, 63] = 2.0
    out, absmax, diag = Q.quantize_c(A, code, 64, 64, 4, True)
    for deq in (Q.dequantize_c, Q.dequantize_np):
        full = deq(out, code, 64, absmax, 64, 4, diag=diag)
        half = deq(out, code, 64, absmax, 64, 4, diag=diag, to_bf16=True)
        expect = torch.from_numpy(full).to(torch.bfloat16).float().numpy()
        assert np.array_equal(half, expect, equal_nan=True)


def test_unsorted_table_is_sorted_and_mapped_back(code_maps):
    code = code_maps[("linear-2", 4)]
    perm = np.random.default_rng(1).permutation(16)
    shuffled = code[perm]
    A = _special_matrix(64, 9)
    A[3, 0] = 0.5
    A[4, 63] = 0.5
    base, am = Q.quantize_c(A, code, 64, 64, 4)
    for fn in (Q.quantize_c, Q.quantize_np, Q.quantize_py):
        out, am2 = fn(A, shuffled, 64, 64, 4)
        idx = Q.unpack_np(out, 4096, 4)
        live = np.repeat(am != 0, 64)                  # all-zero segments get index 0 unmapped
        assert np.array_equal(shuffled[idx][live], code[Q.unpack_np(base, 4096, 4)][live])
        assert np.all(idx[~live] == 0)
        assert np.array_equal(am, am2, equal_nan=True)
    t = QL.quantize_loop(torch.from_numpy(A), torch.from_numpy(shuffled), 64, 64, 4)
    assert np.array_equal(t[0].numpy(), Q.quantize_c(A, shuffled, 64, 64, 4)[0])


# ------------------------------------------------------------------ invariants
@pytest.mark.parametrize("bits,bs", CELLS)
def test_absmax_is_exact_segment_maximum_and_round_trip_is_idempotent(code_maps, bits, bs):
    code = code_maps[("linear-2", bits)]
    order = 192
    A = np.random.default_rng(bits + bs).standard_normal((order, order)).astype(F32)
    out, absmax = Q.quantize_c(A, code, order, bs, bits)
    nb = -(-order // bs)
    for r in (0, 7, order - 1):
        for b in range(nb):
            assert absmax[r * nb + b] == np.abs(A[r, b * bs:(b + 1) * bs]).max()
    back = Q.dequantize_c(out, code, order, absmax, bs, bits)
    # linear-2 has +-1 entries, so every segment's extreme element is reproduced exactly
    # and quantizing the dequantized matrix returns the same codes and scales
    out2, absmax2 = Q.quantize_c(back, code, order, bs, bits)
    assert np.array_equal(absmax, absmax2) and np.array_equal(out, out2)
    err = np.abs(back - A)
    scale = np.repeat(absmax.reshape(order, nb), bs, axis=1)[:, :order]
    half_gap = np.diff(code).max() / 2
    assert np.all(err <= scale * half_gap * (1 + 1e-6))


def test_error_paths():
    code = np.linspace(-1, 1, 16, dtype=F32)
    A = np.zeros((4, 4), F32)
    with pytest.raises(ValueError):
        Q.quantize_np(A, code, 4, 64, 5)
    with pytest.raises(ValueError):
        Q.quantize_c(np.zeros(15, F32), code, 4, 64, 4)
    with pytest.raises(ValueError):
        Q.dequantize_c(np.zeros(8, np.uint8), code, 4, np.zeros(3, F32), 64, 4)
    with pytest.raises(ValueError):
        Q.dequantize_np(np.zeros(8, np.uint8), code, 4, np.zeros(4, F32), 64, 4, diag=np.zeros(3, F32))
