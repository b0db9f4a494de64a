"""GPU parity of the blockwise quantizer: libqtensor_hip.so (through qtensor.functional's
ctypes binding) against the C oracle on identical seeded inputs.  Bit-exact everywhere:
packed codes, fp32 maxima, diagonals and dequantized tensors."""
import numpy as np
import pytest
import torch

from oracle import quant_np as Q

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def F():
    import qtensor.functional as fn
    assert torch.cuda.is_available(), "these tests need the GPU"
    assert fn.lib is not None, "libqtensor_hip.so must be built and loadable on the GPU box"
    return fn


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_bits_equal(got: np.ndarray, want: np.ndarray, what: str):
    """Bit-for-bit on fp32 (so -0.0 != +0.0); any NaN equals any NaN."""
    got = np.ascontiguousarray(got, dtype=F32).reshape(-1)
    want = np.ascontiguousarray(want, dtype=F32).reshape(-1)
    assert got.shape == want.shape, what
    both_nan = np.isnan(got) & np.isnan(want)
    same = (got.view(np.uint32) == want.view(np.uint32)) | both_nan
    if not same.all():
        bad = np.flatnonzero(~same)
        raise AssertionError(f"{what}: {bad.size} of {got.size} differ, first at {bad[0]}: "
                             f"got {got[bad[0]]!r} want {want[bad[0]]!r}")


def run_case(F, A32: np.ndarray, code: np.ndarray, order, bs, bits, diag, dtype):
    """Quantize + dequantize on the GPU and through the oracle; compare everything."""
    if dtype == "bf16":
        A32 = Q.bf16_bits_to_f32(Q.f32_to_bf16_bits(A32.reshape(-1))).reshape(order, order)
        A_dev = dev(A32).to(torch.bfloat16)
        assert np.array_equal(A_dev.float().cpu().numpy(), A32, equal_nan=True)
    else:
        A_dev = dev(A32)
    code_dev = dev(code)
    tag = f"order={order} bs={bs} bits={bits} diag={diag} dtype={dtype}"
    print("case", tag, flush=True)
    if diag:
        out, absmax, dg = F.quantize_blockwise_diagreal(A_dev, code_dev, order, blocksize=bs, bits=bits)
        o_out, o_absmax, o_dg = Q.quantize_c(A32, code, order, bs, bits, True)
        assert_bits_equal(dg.cpu().numpy(), o_dg, tag + " diag")
    else:
        out, absmax = F.quantize_blockwise(A_dev, code_dev, order, blocksize=bs, bits=bits)
        o_out, o_absmax = Q.quantize_c(A32, code, order, bs, bits, False)
        dg, o_dg = None, None
    torch.cuda.synchronize()
    assert_bits_equal(absmax.cpu().numpy(), o_absmax, tag + " absmax")
    got = out.cpu().numpy()
    if not np.array_equal(got, o_out):
        bad = np.flatnonzero(got != o_out)
        raise AssertionError(f"{tag} codes: {bad.size} of {got.size} bytes differ, first at byte {bad[0]}: "
                             f"got {got[bad[0]]:#x} want {o_out[bad[0]]:#x}")
    for outdtype in (torch.float32, torch.bfloat16):
        if diag:
            back = F.dequantize_blockwise_diagreal(out, code_dev, order, absmax, dg, outdtype=outdtype,
                                                   blocksize=bs, bits=bits)
        else:
            back = F.dequantize_blockwise(out, code_dev, order, absmax, outdtype=outdtype, blocksize=bs, bits=bits)
        assert back is not None and back.shape == (order, order) and back.dtype == outdtype
        want = Q.dequantize_c(o_out, code, order, o_absmax, bs, bits, diag=o_dg, to_bf16=outdtype == torch.bfloat16)
        assert_bits_equal(back.float().cpu().numpy(), want, f"{tag} dequant->{outdtype}")


def special_matrix(order, seed):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((order, order)).astype(F32)
    A[rng.random((order, order)) < 0.05] = 0.0
    if order >= 16:
        A[1, :] = 0.0
        A[2, : order // 2] *= F32(1e-41)      # denormals (exact route: maximum below 2^-60)
        A[3, 0] = np.inf
        A[4, order - 1] = np.nan
        A[5, :] *= F32(1e30)                  # maximum above 2^60
        A[6, 1] = -0.0
        A[7, :] *= F32(1e-25)
        A[8, ::3] *= F32(1e-30)               # tiny quotients next to ordinary ones
        A[9, :] = 0.0
        A[9, 9] = 2.5                         # only the diagonal is nonzero
    return A


# ---------------------------------------------------------------------------- arithmetic shortcut
def test_fast_division_equals_ieee_division_for_every_divisor(F):
    """The flat path divides by the segment maximum with rcp + one Newton step and two fmas.  On
    this GPU that must equal IEEE division: exhaustively for the reciprocal (all 1,006,632,961
    fp32 values in [2^-60, 2^60]) and for billions of numerator/denominator pairs."""
    import ctypes as ct
    fn = F.lib.qtensor_hip_check_fast_division
    fn.restype = None
    fn.argtypes = [ct.c_uint32, ct.c_uint32, ct.c_uint32, ct.c_int, ct.c_void_p, ct.c_void_p]
    counts = torch.zeros(3, dtype=torch.int64, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    fn(0x21800000, 0x5d800000, 1, 0, counts.data_ptr(), stream)                # every divisor
    for exp in (67, 100, 126, 127, 128, 187):                                  # whole binades, 64 x each
        fn(exp << 23, (exp << 23) | 0x7fffff if exp < 187 else 0x5d800000, 1, 64, counts.data_ptr(), stream)
    fn(0x21800000, 0x5d800000, 61, 32, counts.data_ptr(), stream)              # sparse sweep of the range
    torch.cuda.synchronize()
    assert F.lib.qtensor_hip_last_error() == 0
    bad_rcp, bad_quot, tried = counts.tolist()
    assert tried > 3_000_000_000
    assert bad_rcp == 0 and bad_quot == 0
    fn(0x21800000 - 1, 0x5d800000, 1, 0, counts.data_ptr(), stream)            # out of range: refused
    assert F.lib.qtensor_hip_last_error() != 0


# ---------------------------------------------------------------------------- C1
def test_config1_orthogonal_1024(F, code_maps):
    g = torch.Generator().manual_seed(0)
    Qm, _ = torch.linalg.qr(torch.randn(1024, 1024, generator=g))
    run_case(F, Qm.numpy().copy(), code_maps[("linear-2", 4)], 1024, 64, 4, False, "fp32")


# ---------------------------------------------------------------------------- cell matrix
CELLS = [(4, 64), (4, 128), (4, 256), (4, 512), (4, 1024), (4, 2048),
         (8, 64), (8, 128), (8, 256), (8, 512), (8, 1024), (8, 2048)]


@pytest.mark.parametrize("bits,bs", CELLS)
@pytest.mark.parametrize("diag", [False, True])
def test_flat_path_all_blocksizes(F, code_maps, bits, bs, diag):
    order = max(bs, 256) * 2 if bs < 2048 else 2048
    for name in ("linear-2", "dynamic"):
        A = special_matrix(order, seed=bits * 1000 + bs)
        run_case(F, A, code_maps[(name, bits)], order, bs, bits, diag, "fp32")
    run_case(F, special_matrix(order, seed=3), code_maps[("linear-2", bits)], order, bs, bits, diag, "bf16")


@pytest.mark.parametrize("order", [1, 2, 3, 5, 17, 63, 64, 65, 100, 129, 169, 200, 576])
@pytest.mark.parametrize("bits,bs", [(4, 64), (4, 128), (8, 256), (8, 64)])
def test_general_path_ragged_and_odd_orders(F, code_maps, order, bits, bs):
    for diag in (False, True):
        for dtype in ("fp32", "bf16"):
            A = special_matrix(order, seed=order + bits)
            run_case(F, A, code_maps[("linear-2", bits)], order, bs, bits, diag, dtype)
    run_case(F, special_matrix(order, seed=order), code_maps[("dynamic", bits)], order, bs, bits, True, "fp32")


def test_large_flat_path_uses_bucket_table(F, code_maps):
    """>= 2^20 elements switches the quantizer to its bucket-table kernel."""
    for bits, bs, name in ((4, 64, "linear-2"), (8, 256, "dynamic"), (8, 64, "linear-2"), (4, 256, "dynamic")):
        order = 1536
        A = special_matrix(order, seed=bits + bs)
        for diag in (False, True):
            run_case(F, A, code_maps[(name, bits)], order, bs, bits, diag, "fp32")
    run_case(F, special_matrix(2048, 5), code_maps[("linear-2", 4)], 2048, 64, 4, True, "bf16")


def test_unsorted_and_unusual_tables(F, code_maps):
    rng = np.random.default_rng(12)
    base = code_maps[("linear-2", 4)]
    tables = [base[rng.permutation(16)],
              np.sort(rng.uniform(-1, 1, 16)).astype(F32),
              np.linspace(-1, 1, 16).astype(F32),
              # thresholds crowded next to zero: forces the exact route everywhere
              np.array([-1, -1e-12, -1e-13, 0, 1e-14, 1e-13, 1e-12, 1e-6, 1e-3, .1, .2, .3, .5, .7, .9, 1], F32)]
    for t in tables:
        for order in (128, 1024):
            A = special_matrix(order, seed=order)
            A[10, :64] = np.array([1e-13, -1e-13, 3e-14, 1.0] * 16, F32)
            run_case(F, A, t, order, 64, 4, False, "fp32")
    t8 = code_maps[("dynamic", 8)][rng.permutation(256)]
    run_case(F, special_matrix(1024, 8), t8, 1024, 256, 8, True, "fp32")


def test_ties_and_exact_codes_on_device(F, code_maps):
    from fractions import Fraction
    for name, bits in (("linear-2", 4), ("linear-2", 8), ("dynamic", 8)):
        code = code_maps[(name, bits)]
        order = 1024
        A = np.zeros((order, order), F32)
        A[:, 0::64] = 1.0
        # every representable exact midpoint, and its two neighbours in fp32
        col = 1
        row = 0
        for i in range(len(code) - 1):
            mid = (Fraction(float(code[i])) + Fraction(float(code[i + 1]))) / 2
            v = F32(float(mid))
            for cand in (v, np.nextafter(v, F32(2)), np.nextafter(v, F32(-2))):
                A[row, col] = cand
                col += 1
                if col % 64 == 0:
                    col += 1
                if col >= order:
                    row, col = row + 1, 1
        for s in range(-(-len(code) // 63)):             # every table entry as an exact input
            part = code[63 * s: 63 * s + 63]
            A[500, 64 * s + 1: 64 * s + 1 + len(part)] = part
        run_case(F, A, code, order, 64, bits, False, "fp32")


# ---------------------------------------------------------------------------- C2
@pytest.mark.parametrize("n", [64, 128, 256, 512, 576, 1024, 1152, 2304])
def test_config2_psd_blocks(F, code_maps, n):
    g = torch.Generator().manual_seed(n)
    A = torch.randn(n, n, generator=g)
    M = (A @ A.T / n + 1e-4 * torch.eye(n)).numpy().copy()
    for diag in (False, True):
        run_case(F, M, code_maps[("linear-2", 4)], n, 64, 4, diag, "fp32")
        run_case(F, M, code_maps[("dynamic", 8)], n, 256, 8, diag, "fp32")


# ---------------------------------------------------------------------------- buffers, errors
def test_buffer_reuse_and_error_paths(F, code_maps):
    code = dev(code_maps[("linear-2", 4)])
    A = torch.randn(256, 256, device="cuda")
    out, absmax, diag = F.quantize_blockwise_diagreal(A, code, 256, blocksize=64, bits=4)
    p = (out.data_ptr(), absmax.data_ptr(), diag.data_ptr())
    B = torch.randn(256, 256, device="cuda")
    out2, absmax2, diag2 = F.quantize_blockwise_diagreal(B, code, 256, absmax=absmax, diag=diag, out=out,
                                                         blocksize=64, bits=4)
    assert (out2.data_ptr(), absmax2.data_ptr(), diag2.data_ptr()) == p
    want = Q.quantize_c(B.cpu().numpy(), code.cpu().numpy(), 256, 64, 4, True)
    assert np.array_equal(out2.cpu().numpy(), want[0])
    with pytest.raises(ValueError):
        F.quantize_blockwise(A.double(), code, 256, blocksize=64, bits=4)
    with pytest.raises(ValueError):
        F.dequantize_blockwise(out, code, 256, absmax[:-1], blocksize=64, bits=4)
    with pytest.raises(ValueError):
        F.dequantize_blockwise(out, code, 256, absmax, outdtype=torch.float16, blocksize=64, bits=4)
    with pytest.raises(AssertionError):
        F.quantize_blockwise(A, code, 256, blocksize=96, bits=4)
    with pytest.raises(AssertionError):
        F.quantize_blockwise(A, code, 256, blocksize=64, bits=8)      # table has 16 entries
    with pytest.raises(RuntimeError):
        F.quantize_blockwise(A.cpu(), code.cpu(), 256, blocksize=64, bits=4)
    # the raw C entry point reports a bad blocksize instead of launching
    F.lib.cquantize_blockwise_4bit_fp32(F.get_ptr(A), F.get_ptr(code), 256, F.get_ptr(absmax), F.get_ptr(out), 96)
    assert F.lib.qtensor_hip_last_error() != 0
    F.lib.cquantize_blockwise_4bit_fp32(F.get_ptr(A), F.get_ptr(code), 256, F.get_ptr(absmax), F.get_ptr(out), 64)
    torch.cuda.synchronize()
    assert F.lib.qtensor_hip_last_error() == 0
    assert np.array_equal(out.cpu().numpy(), Q.quantize_c(A.cpu().numpy(), code.cpu().numpy(), 256, 64, 4)[0])


def test_side_stream_launch(F, code_maps):
    code = dev(code_maps[("linear-2", 4)])
    A = torch.randn(1024, 1024, device="cuda")
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        out, absmax = F.quantize_blockwise(A, code, 1024, blocksize=64, bits=4)
        back = F.dequantize_blockwise(out, code, 1024, absmax, blocksize=64, bits=4)
    s.synchronize()
    o_out, o_absmax = Q.quantize_c(A.cpu().numpy(), code.cpu().numpy(), 1024, 64, 4)
    assert np.array_equal(out.cpu().numpy(), o_out)
    assert_bits_equal(back.cpu().numpy(), Q.dequantize_c(o_out, code.cpu().numpy(), 1024, o_absmax, 64, 4), "stream")


# ---------------------------------------------------------------------------- C5 at full size
def _stress_tensor(order, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(order, order, device="cuda", generator=g)
    mask = torch.rand(order, order, device="cuda", generator=g) < 0.01
    x[mask] *= 10.0
    return x


@pytest.mark.parametrize("bits,bs,name", [(4, 64, "linear-2"), (4, 256, "linear-2"), (8, 64, "dynamic"), (8, 256, "dynamic")])
def test_config5_full_size_slices_and_invariants(F, code_maps, bits, bs, name):
    order = 16384
    code = code_maps[(name, bits)]
    code_dev = dev(code)
    x = _stress_tensor(order)
    out, absmax = F.quantize_blockwise(x, code_dev, order, blocksize=bs, bits=bits)
    back = F.dequantize_blockwise(out, code_dev, order, absmax, blocksize=bs, bits=bits)
    torch.cuda.synchronize()
    # whole-tensor invariants: maxima are exact; error bounded by half the widest gap
    seg_max = x.view(-1, bs).abs().amax(dim=1)
    assert torch.equal(seg_max, absmax)
    # (a table without -1, like the dynamic one, clamps the negative extreme to its first entry)
    gap = max(float(np.diff(code).max()) / 2, 1 + float(code[0]), 1 - float(code[-1])) + 2e-7   # + fp32 rounding of code*absmax
    assert bool(((back - x).abs().view(-1, bs) <= seg_max[:, None] * gap).all())
    if name == "linear-2":   # table holds +-1: requantizing the result is the identity
        out2, absmax2 = F.quantize_blockwise(back, code_dev, order, blocksize=bs, bits=bits)
        assert torch.equal(out2, out) and torch.equal(absmax2, absmax)
    # bit-exact on 4,194,304-element slices: 256 consecutive rows re-viewed as 2048 x 2048
    per_byte = 8 // bits
    for row0 in (0, 7168, order - 256):
        off = row0 * order
        sl = x.view(-1)[off: off + 2048 * 2048].cpu().numpy()
        o_out, o_absmax = Q.quantize_c(sl, code, 2048, bs, bits)
        assert np.array_equal(out[off // per_byte: (off + 2048 * 2048) // per_byte].cpu().numpy(), o_out)
        assert_bits_equal(absmax[off // bs: (off + 2048 * 2048) // bs].cpu().numpy(), o_absmax, "slice absmax")
        want = Q.dequantize_c(o_out, code, 2048, o_absmax, bs, bits)
        assert_bits_equal(back.view(-1)[off: off + 2048 * 2048].cpu().numpy(), want, "slice dequant")


def test_config5_whole_tensor_against_oracle(F, code_maps):
    """All 268M elements of the headline case (4-bit, block 64) against the C oracle."""
    order = 16384
    code = code_maps[("linear-2", 4)]
    x = _stress_tensor(order, seed=1)
    out, absmax = F.quantize_blockwise(x, dev(code), order, blocksize=64, bits=4)
    torch.cuda.synchronize()
    o_out, o_absmax = Q.quantize_c(x.cpu().numpy(), code, order, 64, 4)
    assert np.array_equal(out.cpu().numpy(), o_out)
    assert_bits_equal(absmax.cpu().numpy(), o_absmax, "absmax")
