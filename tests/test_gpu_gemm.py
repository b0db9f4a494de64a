"""GPU parity of the fused matrix-core products (qtensor.fused.gemm -> qtensor_hip_gemm).

Reference for every case: dequantize with the CPU oracle, multiply in float64 on the CPU.
Tolerance: relative Frobenius error <= 1e-5 (fp32 products accumulate in fp32 on the matrix
cores; observed errors are around 1e-7)."""
import numpy as np
import pytest
import torch

from oracle import quant_np as Q

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def mods():
    import qtensor.functional as F
    import qtensor.fused as X
    assert torch.cuda.is_available() and F.lib is not None
    return F, X


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    want = want.double()
    return float((got.detach().cpu().double() - want).norm() / want.norm().clamp_min(1e-300))


def make_quantized(F, X, mats: torch.Tensor, code: np.ndarray, bits, bs, diag):
    """Quantize a [batch, n, n] stack on the GPU into stacked buffers; also returns the oracle's
    dequantized float64 copy of the same codes."""
    batch, n, _ = mats.shape
    code_d = torch.from_numpy(code).cuda()
    codes = torch.empty(batch, n * n * bits // 8, dtype=torch.uint8, device="cuda")
    absmax = torch.empty(batch, n * n // bs, dtype=torch.float32, device="cuda")
    dg = torch.empty(batch, n, dtype=torch.float32, device="cuda") if diag else None
    deq = []
    for b in range(batch):
        m = mats[b].contiguous().cuda()
        if diag:
            F.quantize_blockwise_diagreal(m, code_d, n, absmax=absmax[b], diag=dg[b], out=codes[b], blocksize=bs, bits=bits)
        else:
            F.quantize_blockwise(m, code_d, n, absmax=absmax[b], out=codes[b], blocksize=bs, bits=bits)
        o = Q.quantize_c(mats[b].numpy(), code, n, bs, bits, diag)
        assert np.array_equal(codes[b].cpu().numpy(), o[0])
        deq.append(Q.dequantize_c(o[0], code, n, o[1], bs, bits, diag=o[2] if diag else None))
    q = X.Quantized(codes, absmax, dg, n, bs, bits, code_d)
    return q, torch.from_numpy(np.stack(deq)).double()


@pytest.mark.parametrize("m,n,k,batch", [(128, 128, 128, 1), (64, 64, 16, 3), (100, 65, 33, 2), (257, 129, 70, 1),
                                         (768, 3072, 768, 1), (1024, 1024, 1024, 2), (1, 1, 1, 1), (300, 5, 1000, 1)])
def test_dense_products_all_layouts(mods, m, n, k, batch):
    _, X = mods
    g = torch.Generator().manual_seed(m * 7 + n)
    A = torch.randn(batch, m, k, generator=g)
    B = torch.randn(batch, k, n, generator=g)
    want = A.double() @ B.double()
    Ad, Bd = A.cuda(), B.cuda()
    assert rel_err(X.gemm(Ad, Bd), want) <= TOL
    assert rel_err(X.gemm(Ad.transpose(1, 2).contiguous(), Bd, trans_a=True), want) <= TOL
    assert rel_err(X.gemm(Ad, Bd.transpose(1, 2).contiguous(), trans_b=True), want) <= TOL
    # views with a larger leading dimension and an unaligned start
    big = torch.zeros(batch, m + 3, k + 5, device="cuda")
    big[:, 1:m + 1, 1:k + 1] = Ad
    assert rel_err(X.gemm(big[:, 1:m + 1, 1:k + 1], Bd), want) <= TOL
    if batch == 1:
        out2 = X.gemm(Ad[0], Bd[0])
        assert out2.shape == (m, n) and rel_err(out2, want[0]) <= TOL


@pytest.mark.parametrize("bits,bs,name", [(4, 64, "linear-2"), (8, 256, "dynamic"), (8, 64, "linear-2"), (4, 128, "dynamic")])
@pytest.mark.parametrize("diag", [False, True])
def test_quantized_factor_times_dense(mods, code_maps, bits, bs, name, diag):
    F, X = mods
    g = torch.Generator().manual_seed(bits + bs)
    # (few and many matrices, narrow and wide partners: between them the cases take every tile shape)
    for n, other, batch in ((256, 100, 2), (768, 320, 1), (1024, 64, 1), (256, 200, 40), (512, 128, 24), (128, 64, 60), (64, 256, 30)):
        if n % bs:
            continue
        mats = torch.randn(batch, n, n, generator=g)
        mats[:, 3, :64] = 0.0                                  # a zero-maximum segment
        q, deq = make_quantized(F, X, mats, code_maps[(name, bits)], bits, bs, diag)
        G_left = torch.randn(batch, n, other, generator=g)
        G_right = torch.randn(batch, other, n, generator=g)
        for pipe in ("split", "f32"):                          # chosen per product: the process-wide mode stays as it is
            assert rel_err(X.gemm(q, G_left.cuda(), pipe=pipe), deq @ G_left.double()) <= TOL, (pipe, n, other, batch)
            assert rel_err(X.gemm(G_right.cuda(), q, pipe=pipe), G_right.double() @ deq) <= TOL, (pipe, n, other, batch)


def test_config3_preconditioned_gradient(mods, code_maps):
    """G 768 x 3072 ~ N(0, 0.02^2); L (768) and R (3072) are inverse 4th roots of seeded PSD matrices with
    eigenvalues log-uniform in [1e-6, 1], stored 4-bit / block 64 with exact diagonal."""
    F, X = mods
    code = code_maps[("linear-2", 4)]
    g = torch.Generator().manual_seed(3)

    def inv_root(n):
        qm, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
        lam = 10.0 ** (-6 * torch.rand(n, generator=g, dtype=torch.float64))
        return ((qm * lam ** -0.25) @ qm.T).float()

    L, R = inv_root(768), inv_root(3072)
    G = 0.02 * torch.randn(768, 3072, generator=g)
    for diag in (True, False):
        Lq, Ld = make_quantized(F, X, L[None], code, 4, 64, diag)
        Rq, Rd = make_quantized(F, X, R[None], code, 4, 64, diag)
        want = Ld[0] @ G.double() @ Rd[0]
        got = X.precondition(G.cuda(), Lq, Rq)
        assert got.shape == (768, 3072)
        assert rel_err(got, want) <= TOL
        # and equal, to the same tolerance, to dequantize-then-matmul on the device
        Lg = F.dequantize_blockwise_diagreal(Lq.codes[0], Lq.code, 768, Lq.absmax[0], Lq.diag[0], blocksize=64, bits=4) if diag \
            else F.dequantize_blockwise(Lq.codes[0], Lq.code, 768, Lq.absmax[0], blocksize=64, bits=4)
        assert torch.equal(Lg.cpu().double(), Ld[0])
        Rg = torch.from_numpy(Rd[0].numpy().astype(np.float32)).cuda()
        assert rel_err(got, (Lg @ G.cuda() @ Rg).cpu()) <= TOL


@pytest.mark.parametrize("m,n", [(256, 512), (768, 1024), (100, 260), (1024, 768), (101, 330), (2, 131)])
def test_gram_and_statistics_update(mods, code_maps, m, n):
    F, X = mods
    g = torch.Generator().manual_seed(m + n)
    G = 0.02 * torch.randn(2, m, n, generator=g)
    Gd = G.cuda()
    assert rel_err(X.gram(Gd, 0), G.double() @ G.double().transpose(1, 2)) <= TOL
    assert rel_err(X.gram(Gd, 1), G.double().transpose(1, 2) @ G.double()) <= TOL
    beta = 0.95
    for axis, order in ((0, m), (1, n)):
        S = (G.double() @ G.double().transpose(1, 2)) if axis == 0 else (G.double().transpose(1, 2) @ G.double())
        old = torch.randn(2, order, order, generator=g) * 1e-3
        old = old @ old.transpose(1, 2) + 1e-6 * torch.eye(order)
        assert rel_err(X.gram(Gd, axis, stat=old.cuda(), beta=beta, alpha=1 - beta), beta * old.double() + (1 - beta) * S) <= TOL
        if order % 64 == 0:
            q, deq = make_quantized(F, X, old, code_maps[("linear-2", 4)], 4, 64, True)
            assert rel_err(X.gram(Gd, axis, stat=q, beta=beta, alpha=1 - beta), beta * deq + (1 - beta) * S) <= TOL


def test_newton_epilogue_and_skip_flags(mods):
    _, X = mods
    g = torch.Generator().manual_seed(9)
    n, batch = 192, 3
    A = torch.randn(batch, n, n, generator=g) / n ** 0.5
    B = torch.randn(batch, n, n, generator=g) / n ** 0.5
    want = A.double() @ B.double()
    w = -0.25
    out = torch.full((batch, n, n), 7.0, device="cuda")
    T = torch.full((batch, n, n), 7.0, device="cuda")
    err = torch.zeros(batch, device="cuda")
    skip = torch.tensor([0, 1, 0], dtype=torch.int32, device="cuda")
    X.gemm(A.cuda(), B.cuda(), out=out, newton=(T, w, err), skip=skip)
    eye = torch.eye(n, dtype=torch.float64)
    for b in (0, 2):
        assert rel_err(out[b], want[b]) <= TOL
        assert rel_err(T[b], (1 - w) * eye + w * want[b]) <= TOL
        assert abs(float(err[b]) - float((want[b] - eye).abs().max())) <= 1e-5
    assert bool((out[1] == 7.0).all()) and bool((T[1] == 7.0).all()) and float(err[1]) == 0.0


@pytest.mark.parametrize("n,batch", [(192, 3), (1024, 2), (150, 2), (77, 1)])
def test_symmetric_products_compute_the_upper_half_and_mirror_it(mods, n, batch):
    """Products of commuting symmetric matrices (the Newton iterates of a symmetric statistic)."""
    _, X = mods
    g = torch.Generator().manual_seed(n)
    S = torch.randn(batch, n, n, generator=g) / n ** 0.5
    S = (S + S.transpose(1, 2)) / 2
    P = (S @ S + 0.5 * S).contiguous()                           # a polynomial in S: commutes with S
    P = ((P + P.transpose(1, 2)) / 2).contiguous()
    want = S.double() @ P.double()
    w = -0.25
    out = torch.full((batch, n, n), 7.0, device="cuda")
    T = torch.full((batch, n, n), 7.0, device="cuda")
    err = torch.zeros(batch, device="cuda")
    skip = torch.zeros(batch, dtype=torch.int32, device="cuda")
    skip[-1] = 1 if batch > 1 else 0
    X.gemm(S.cuda(), P.cuda(), out=out, newton=(T, w, err), skip=skip, symmetric=True)
    eye = torch.eye(n, dtype=torch.float64)
    for b in range(batch):
        if int(skip[b]):
            assert bool((out[b] == 7.0).all()) and bool((T[b] == 7.0).all()) and float(err[b]) == 0.0
            continue
        # the float64 product is symmetric only up to the non-commutation left by rounding P
        assert rel_err(out[b], (want[b] + want[b].T) / 2) <= TOL
        assert rel_err(T[b], (1 - w) * eye + w * (want[b] + want[b].T) / 2) <= TOL
        assert abs(float(err[b]) - float((want[b] - eye).abs().max())) <= 1e-5
        tile = torch.arange(n) // 128                           # tiles are 64 or 128 wide: this holds for both
        off = tile[:, None] != tile[None, :]                    # outside the diagonal tiles: exact mirror
        o = out[b].cpu()
        assert torch.equal(o[off], o.T[off])
    plain = X.gemm(S.cuda(), P.cuda())
    sym = X.gemm(S.cuda(), P.cuda(), symmetric=True)
    upper = torch.arange(n)[:, None] <= torch.arange(n)[None, :]
    # on and above the diagonal both modes run the same arithmetic (below it the symmetric mode mirrors: tile by tile,
    # and on the split pipe inside the diagonal tiles as well)
    if n <= 192:
        assert torch.equal(plain.cpu()[:, upper], sym.cpu()[:, upper])
    with pytest.raises(ValueError):
        X.gemm(torch.zeros(64, 32, device="cuda"), torch.zeros(32, 48, device="cuda"), symmetric=True)


def test_argument_errors(mods, code_maps):
    F, X = mods
    A = torch.randn(64, 32, device="cuda")
    with pytest.raises(ValueError):
        X.gemm(A, torch.randn(31, 8, device="cuda"))
    with pytest.raises(ValueError):
        X.gemm(A.double(), A.double().T)
    with pytest.raises(ValueError):
        X.gemm(A.cpu(), A.cpu().T.contiguous())
    q, _ = make_quantized(F, X, torch.randn(1, 128, 128), code_maps[("linear-2", 4)], 4, 64, True)
    with pytest.raises(RuntimeError):                           # two quantized factors: not built
        X.gemm(q, q)
    with pytest.raises(ValueError):
        X.gemm(q, torch.randn(64, 8, device="cuda"))


@pytest.mark.parametrize("bits,bs,name,n,batch", [(4, 64, "linear-2", 768, 5), (4, 64, "linear-2", 64, 33),
                                                   (8, 256, "dynamic", 512, 3), (4, 128, "dynamic", 128, 7)])
def test_stack_quantize_dequantize_equal_per_matrix_calls(mods, code_maps, bits, bs, name, n, batch):
    F, X = mods
    g = torch.Generator().manual_seed(n + batch)
    mats = torch.randn(batch, n, n, generator=g)
    mats[1, 2, :] = 0.0
    code = code_maps[(name, bits)]
    code_d = torch.from_numpy(code).cuda()
    for diag in (False, True):
        for dtype in (torch.float32, torch.bfloat16):
            src = mats.to(dtype)
            q = X.quantize_stack(src.cuda(), X.empty_quantized(batch, n, bs, bits, code_d, diag))
            back = X.dequantize_stack(q)
            back16 = X.dequantize_stack(q, outdtype=torch.bfloat16)
            torch.cuda.synchronize()
            for b in range(batch):
                o = Q.quantize_c(src[b].float().numpy(), code, n, bs, bits, diag)
                assert np.array_equal(q.codes[b].cpu().numpy(), o[0])
                assert np.array_equal(q.absmax[b].cpu().numpy(), o[1])
                if diag:
                    assert np.array_equal(q.diag[b].cpu().numpy(), o[2])
                want = Q.dequantize_c(o[0], code, n, o[1], bs, bits, diag=o[2] if diag else None)
                assert np.array_equal(back[b].cpu().numpy(), want)
                want16 = Q.dequantize_c(o[0], code, n, o[1], bs, bits, diag=o[2] if diag else None, to_bf16=True)
                assert np.array_equal(back16[b].float().cpu().numpy(), want16)


@pytest.mark.parametrize("bits,bs,name,n,batch", [(4, 64, "linear-2", 768, 3), (4, 64, "linear-2", 64, 9), (8, 64, "linear-2", 192, 2),
                                                   (8, 256, "dynamic", 512, 3), (4, 128, "dynamic", 384, 2), (4, 256, "linear-2", 256, 2)])
def test_quantizer_reading_the_transpose_equals_the_oracle_on_the_transposed_matrix(mods, code_maps, bits, bs, name, n, batch):
    """quantize_stack(..., transposed=True) never writes the transpose; codes and maxima must be the oracle's for
    mats[b].T bit for bit, including zero segments, tiny / huge / NaN maxima (exact-division route) and a
    table handed over in descending order."""
    F, X = mods
    g = torch.Generator().manual_seed(7 * n + batch)
    mats = torch.randn(batch, n, n, generator=g)
    mats[0, :64, 3] = 0.0                                        # a zero segment of row 3 of the transpose
    mats[0, :64, 5] *= 1e-30                                     # maxima outside the fast-division range
    mats[0, :64, 6] *= 1e30
    mats[batch - 1, 10, 7] = float("nan")
    for code in (code_maps[(name, bits)], code_maps[(name, bits)][::-1].copy()):
        code_d = torch.from_numpy(code).cuda()
        q = X.quantize_stack(mats.cuda(), X.empty_quantized(batch, n, bs, bits, code_d, False), transposed=True)
        torch.cuda.synchronize()
        for b in range(batch):
            o = Q.quantize_c(mats[b].T.contiguous().numpy(), code, n, bs, bits, False)
            assert np.array_equal(q.codes[b].cpu().numpy(), o[0])
            assert np.array_equal(q.absmax[b].cpu().numpy(), o[1], equal_nan=True)
    # forms the kernel does not take go through a transposed copy and the ordinary quantizer
    code = code_maps[(name, bits)]
    code_d = torch.from_numpy(code).cuda()
    q = X.quantize_stack(mats.cuda(), X.empty_quantized(batch, n, bs, bits, code_d, True), transposed=True)
    o = Q.quantize_c(mats[0].T.contiguous().numpy(), code, n, bs, bits, True)
    assert np.array_equal(q.codes[0].cpu().numpy(), o[0]) and np.array_equal(q.diag[0].cpu().numpy(), o[2])


@pytest.mark.parametrize("bits,name,n,k,batch,diag", [(4, "linear-2", 768, 256, 3, True), (4, "linear-2", 320, 100, 2, True),
                                                       (8, "dynamic", 256, 512, 2, True), (4, "dynamic", 128, 64, 5, False),
                                                       (4, "linear-2", 64, 32, 4, True)])
@pytest.mark.parametrize("pipe", ["f32", "split"])
def test_statistics_update_encoded_in_place_equals_update_then_quantize_bit_for_bit(mods, code_maps, bits, name, n, k, batch, diag, pipe):
    """L <- beta L + (1 - beta) G G^T (and G^T G) with the result re-encoded inside the product's epilogue: codes,
    maxima and exact diagonal must be those of the two-step path (fused product to fp32, then the stack quantizer,
    which the other tests pin to the oracle) -- including zero, tiny, huge and NaN segments.

    On both matrix pipes.  (On the split pipe a b and b a add the pieces of a product in different orders; symmetric
    products there give every element below the diagonal the value of its partner above, whatever the tile shape,
    so the two paths -- whose tile shapes differ -- still agree bit for bit, mirrored or multiplied out.)"""
    F, X = mods
    before = X.gemm_pipe(pipe)
    try:
        _encoded_in_place_case(X, code_maps, bits, name, n, k, batch, diag)
    finally:
        X.gemm_pipe(before)


def _encoded_in_place_case(X, code_maps, bits, name, n, k, batch, diag):
    g = torch.Generator().manual_seed(n + k)
    code = code_maps[(name, bits)]
    code_d = torch.from_numpy(code).cuda()
    L0 = torch.randn(batch, n, n, generator=g)
    L0 = (L0 @ L0.transpose(1, 2) / n).contiguous()
    for side in (0, 1):
        G = (0.3 * torch.randn(batch, n, k, generator=g)) if side == 0 else (0.3 * torch.randn(batch, k, n, generator=g))
        if side == 0:
            G[0, 5, :] = 0.0                      # row/column 5 of G G^T is zero
            G[batch - 1, 7, 3] = float("nan")
            G[1, 9, :] *= 1e-22                   # maxima below the fast-division range once squared with the addend gone
        Gd = G.cuda()
        for beta in (0.95, 0.0):
            two = X.quantize_stack(L0.cuda(), X.empty_quantized(batch, n, 64, bits, code_d, diag))
            one = X.quantize_stack(L0.cuda(), X.empty_quantized(batch, n, 64, bits, code_d, diag))
            kw = dict(trans_b=True) if side == 0 else dict(trans_a=True)
            half = not (side == 1 and beta == 0.0)          # once with every tile multiplied out
            # (the two-step path likewise: on the split pipe an element multiplied out below the diagonal differs in
            # its last bits from the mirror image of its partner above)
            dense = X.gemm(Gd, Gd, addend=two, alpha=1.0 - beta, beta=beta, symmetric=half, **kw)
            X.quantize_stack(dense, two)
            got = X.gemm(Gd, Gd, addend=one, alpha=1.0 - beta, beta=beta, symmetric=half, requantize=True, **kw)
            torch.cuda.synchronize()
            assert got is one
            assert torch.equal(one.codes, two.codes)
            assert np.array_equal(one.absmax.cpu().numpy(), two.absmax.cpu().numpy(), equal_nan=True)
            if diag:
                assert np.array_equal(one.diag.cpu().numpy(), two.diag.cpu().numpy(), equal_nan=True)
    with pytest.raises(ValueError):
        X.gemm(Gd, Gd, trans_a=True, addend=X.empty_quantized(batch, n, 128, bits, code_d, diag) if n % 128 == 0 else None,
               requantize=True)


@pytest.mark.parametrize("n,rows,batch", [(64, 64, 3), (320, 200, 2), (768, 768, 2)])
def test_products_with_a_triangular_factor_skip_its_zero_part_and_change_nothing(mods, n, rows, batch):
    _, X = mods
    g = torch.Generator().manual_seed(n)
    U = torch.triu(torch.randn(batch, n, n, generator=g))
    Q = torch.randn(batch, rows, n, generator=g)
    W = torch.randn(batch, n, rows, generator=g)
    Ud, Qd, Wd = U.cuda(), Q.cuda(), W.cuda()
    assert rel_err(X.gemm(Qd, Ud, upper_b=True), Q.double() @ U.double()) <= TOL
    assert rel_err(X.gemm(Ud, Wd, upper_a=True), U.double() @ W.double()) <= TOL
    assert rel_err(X.gemm(Ud, Ud, upper_a=True, upper_b=True), U.double() @ U.double()) <= TOL
    E = torch.randn(batch, rows, n, generator=g).cuda()
    assert rel_err(X.gemm(Qd, Ud, upper_b=True, addend=E, alpha=-1.0, beta=0.5), 0.5 * E.cpu().double() - Q.double() @ U.double()) <= TOL
    with pytest.raises(ValueError):
        X.gemm(Qd, torch.zeros(batch, n, n + 64, device="cuda"), upper_b=True)        # not square in its k index


@pytest.mark.parametrize("m,n,k,batch", [(768, 3072, 3072, 1), (256, 256, 2048, 2), (100, 260, 1024, 1)])
def test_products_split_along_k_equal_the_unsplit_ones_to_rounding(mods, m, n, k, batch, monkeypatch):
    """Few output tiles and a long k range: the library cuts k into slices whose partial products go through
    a scratch area and are summed in a fixed order (deterministic: two runs agree bit for bit)."""
    _, X = mods
    g = torch.Generator().manual_seed(k + m)
    A = torch.randn(batch, m, k, generator=g)
    B = torch.randn(batch, k, n, generator=g)
    want = A.double() @ B.double()
    Ad, Bd = A.cuda(), B.cuda()
    first = X.gemm(Ad, Bd)
    assert rel_err(first, want) <= TOL
    assert torch.equal(first, X.gemm(Ad, Bd))
    monkeypatch.setattr(X, "_WORKSPACE_FLOATS", 0)                 # no scratch: no split
    assert rel_err(X.gemm(Ad, Bd), want) <= TOL
    out = torch.full((batch, m, n + 3), 7.0, device="cuda")          # a strided destination keeps its padding
    monkeypatch.setattr(X, "_WORKSPACE_FLOATS", 1 << 24)
    X.gemm(Ad, Bd, out=out[:, :, :n])
    assert rel_err(out[:, :, :n], want) <= TOL and bool((out[:, :, n:] == 7.0).all())


def test_random_shapes_strides_and_alignments_all_dense_layouts(mods):
    """Seeded sweep over odd extents, padded leading dimensions and base addresses that are not 16-byte
    aligned: exercises the predicate-free tile loads, the guarded ones and the switch between them."""
    _, X = mods
    g = torch.Generator().manual_seed(1234)
    pick = lambda choices: choices[int(torch.randint(len(choices), (1,), generator=g))]      # noqa: E731
    for case in range(60):
        m, n = pick([1, 4, 31, 64, 100, 128, 130, 257]), pick([1, 4, 33, 64, 96, 128, 200, 260])
        k = pick([1, 15, 16, 17, 32, 48, 100, 256, 272])
        batch, ta, tb = pick([1, 1, 2, 3]), pick([False, True]), pick([False, True])
        pad_a, pad_b, shift_a, shift_b = pick([0, 0, 4, 3]), pick([0, 0, 4, 1]), pick([0, 0, 1]), pick([0, 0, 2])

        def operand(rows, cols, pad, shift):
            flat = torch.randn(batch * rows * (cols + pad) + shift, generator=g).cuda()
            return flat[shift:].view(batch, rows, cols + pad)[:, :, :cols]

        A = operand(k, m, pad_a, shift_a) if ta else operand(m, k, pad_a, shift_a)
        B = operand(n, k, pad_b, shift_b) if tb else operand(k, n, pad_b, shift_b)
        Ad = A.double().cpu().transpose(1, 2) if ta else A.double().cpu()
        Bd = B.double().cpu().transpose(1, 2) if tb else B.double().cpu()
        want = Ad @ Bd
        if ta and tb:                                  # A^T B^T is not on the path and not built
            with pytest.raises(RuntimeError):
                X.gemm(A, B, trans_a=ta, trans_b=tb)
            continue
        got = X.gemm(A, B, trans_a=ta, trans_b=tb)
        assert got.shape == (batch, m, n)
        assert rel_err(got, want) <= TOL, (case, m, n, k, batch, ta, tb, pad_a, pad_b, shift_a, shift_b)


@pytest.mark.parametrize("shift", [0, 1])
def test_operands_inside_very_wide_arrays_are_read_where_they_are(mods, shift):
    """Dense operands given as views into wide arrays.  The split pipe's loads take a tile's base from scalar registers
    and a byte offset of 32 bits per lane: with a leading dimension just under 2^22 words the offsets of a tile's last
    rows lie beyond 2^31 bytes and must still be taken as unsigned; from 2^22 words on the product goes to the fp32
    pipe.  Results must be those of the same operands stored compactly (bit for bit on the same pipe).  shift 1: rows
    that are not 16-byte aligned (word loads)."""
    _, X = mods
    g = torch.Generator(device="cuda").manual_seed(31 + shift)
    a = torch.randn(128, 64, device="cuda", generator=g)
    b = torch.randn(64, 128, device="cuda", generator=g)
    want = a.double().cpu() @ b.double().cpu()
    compact = X.gemm(a, b)
    assert rel_err(compact, want) <= TOL
    for ld, same_pipe in (((1 << 22) - 4, True), (1 << 22, False)):
        wide_a = torch.zeros(128, ld, device="cuda")
        wide_b = torch.zeros(64, ld, device="cuda")
        A = wide_a[:, 1000 + shift:1064 + shift]
        B = wide_b[:, 2000 + shift:2128 + shift]
        A.copy_(a)
        B.copy_(b)
        got = X.gemm(A, B)                                   # A: k contiguous, B: row index contiguous
        assert torch.equal(got, compact) if same_pipe else rel_err(got, want) <= TOL
        for got_t, compact_t in ((X.gemm(B, b, trans_a=True), X.gemm(b, b, trans_a=True)),        # left operand with its row index contiguous
                                 (X.gemm(a, A, trans_b=True), X.gemm(a, a, trans_b=True))):       # right operand with k contiguous
            assert torch.equal(got_t, compact_t) if same_pipe else rel_err(got_t, compact_t.cpu()) <= TOL
        del wide_a, wide_b, A, B
    torch.cuda.empty_cache()


@pytest.mark.parametrize("batch,m,n,k", [(64, 256, 384, 64), (40, 512, 512, 1024), (6, 1024, 1024, 2048), (50, 500, 392, 336),
                                         (3, 200, 72, 160), (1, 64, 64, 32)])
@pytest.mark.parametrize("spread", [0.0, 3.0])
def test_split_pipe_is_as_accurate_as_the_fp32_pipe(mods, batch, m, n, k, spread):
    """Products of dense operands on the bf16 pipe (each operand split into three bf16 pieces, six products per fp32
    product) against the same products on the fp32 pipe, both measured against float64 element by element in units of
    sum_k |a_ik| |b_kj| (the scale of the rounding errors of a dot product): the split pipe must not be worse -- it
    measures 0.7-0.9 of the fp32 pipe's error, because each MFMA instruction adds sixteen products before it rounds
    where the fp32 instruction adds two.  All three operand layouts, every tile shape (the batch and extents decide
    it), well scaled entries and entries spread over e^(+-9)."""
    _, X = mods
    g = torch.Generator().manual_seed(batch * 7 + k)
    for trans_a, trans_b in ((False, False), (False, True), (True, False)):
        A = torch.randn((batch, k, m) if trans_a else (batch, m, k), generator=g)
        B = torch.randn((batch, n, k) if trans_b else (batch, k, n), generator=g)
        A = (A * torch.exp(spread * torch.randn(A.shape, generator=g))).cuda()
        B = (B * torch.exp(spread * torch.randn(B.shape, generator=g))).cuda()
        a64 = (A.transpose(1, 2) if trans_a else A).double()
        b64 = (B.transpose(1, 2) if trans_b else B).double()
        want, scale = a64 @ b64, a64.abs() @ b64.abs()
        out = {pipe: X.gemm(A, B, trans_a=trans_a, trans_b=trans_b, pipe=pipe) for pipe in ("f32", "split")}
        assert not torch.equal(out["f32"], out["split"])                     # the split pipe was taken
        err = {p: ((o.double() - want).abs() / scale) for p, o in out.items()}
        assert float(err["split"].max()) <= 1.05 * float(err["f32"].max()) + 1e-8, (trans_a, trans_b)
        assert float(err["split"].mean()) <= 1.02 * float(err["f32"].mean()), (trans_a, trans_b)
        assert float(err["split"].max()) <= 2e-5 and float(err["f32"].max()) <= 2e-5


def test_split_pipe_switch_epilogues_and_special_values(mods):
    _, X = mods
    before = X.gemm_pipe()
    try:
        assert X.gemm_pipe("f32") == before and X.gemm_pipe() == "f32"
        assert X.gemm_pipe("split") == "f32" and X.gemm_pipe() == "split"
        with pytest.raises(ValueError):
            X.gemm_pipe("bf16")
        g = torch.Generator().manual_seed(5)
        B, n = 20, 256
        A, Bm, E = (torch.randn(B, n, n, generator=g).cuda() for _ in range(3))
        # fused epilogue and symmetric mirroring on the split pipe
        got = X.gemm(A, Bm, addend=E, alpha=-0.5, beta=1.5)
        assert rel_err(got, (1.5 * E.double() - 0.5 * (A.double() @ Bm.double())).cpu()) <= TOL
        sym = X.gemm(A, A, trans_b=True, symmetric=True)
        assert rel_err(sym, (A.double() @ A.double().transpose(1, 2)).cpu()) <= TOL
        assert torch.equal(sym, sym.transpose(1, 2))                       # exactly symmetric, diagonal tiles included
        one = X.gemm(A[:1], A[:1], trans_b=True, symmetric=True)           # a single matrix takes smaller tiles: same bits
        assert torch.equal(one[0], sym[0])
        # a k extent that is not a whole number of tiles goes to the fp32 pipe: same bits in both modes
        odd = [X.gemm(A[:, :, :100].contiguous(), Bm[:, :100].contiguous()) for _ in (X.gemm_pipe("f32"), X.gemm_pipe("split"))]
        assert torch.equal(odd[0], odd[1])
        X.gemm_pipe("split")
        # tiny and huge entries keep fp32 accuracy; an infinite entry poisons its row with NaN (the fp32 pipe gives inf)
        tiny = X.gemm(A * 1e-30, Bm * 1e-5)
        assert rel_err(tiny, ((A.double() * 1e-30) @ (Bm.double() * 1e-5)).cpu()) <= TOL
        huge = X.gemm(A * 1e18, Bm * 1e15)
        assert rel_err(huge, ((A.double() * 1e18) @ (Bm.double() * 1e15)).cpu()) <= TOL
        bad = A.clone()
        bad[3, 7, 9] = float("inf")
        out = X.gemm(bad, Bm)
        assert bool(out[3, 7].isnan().all()) and bool(torch.isfinite(out[3, 8]).all()) and bool(torch.isfinite(out[2]).all())
        # the per-product choice overrides the process-wide mode, in both directions, and leaves it alone
        assert torch.equal(X.gemm(A, Bm, pipe="f32"), [X.gemm_pipe("f32"), X.gemm(A, Bm), X.gemm_pipe("split")][1])
        assert torch.equal(X.gemm(A, Bm, pipe="split"), X.gemm(A, Bm)) and X.gemm_pipe() == "split"
        with pytest.raises(ValueError):
            X.gemm(A, Bm, pipe="bf16")
    finally:
        X.gemm_pipe(before)


def test_split_pipe_at_the_top_of_the_fp32_range(mods):
    """The leading bf16 piece of an element rounds to infinity from 0x7f7f8000 (about 3.3962e38) on: such an element
    behaves like an infinite one on the split pipe (NaN in its row of the result), as the header says; just below
    that the product is as accurate as anywhere else, and the fp32 pipe takes the whole range."""
    _, X = mods
    g = torch.Generator().manual_seed(9)
    n = 128
    A = torch.randn(1, n, n, generator=g).cuda()
    Bm = torch.zeros(1, n, n, device="cuda")
    Bm[0].fill_diagonal_(2.0 ** -20)                          # results stay finite: each is one scaled element of A
    below = torch.tensor(0x7f7f7fff, dtype=torch.int32).view(torch.float32).item()      # the largest element that still splits
    at = torch.tensor(0x7f7f8000, dtype=torch.int32).view(torch.float32).item()
    A[0, 5, 17], A[0, 9, 3] = below, -below
    for pipe in ("split", "f32"):
        out = X.gemm(A, Bm, pipe=pipe)
        assert bool(torch.isfinite(out).all())
        assert rel_err(out, (A.double() @ Bm.double()).cpu()) <= TOL
    A[0, 5, 17] = at
    out = X.gemm(A, Bm, pipe="split")
    assert bool(out[0, 5].isnan().all()) and bool(torch.isfinite(out[0, 4]).all()) and bool(torch.isfinite(out[0, 9]).all())
    assert bool(torch.isfinite(X.gemm(A, Bm, pipe="f32")).all())


@pytest.mark.parametrize("m,n,k,batch", [(17, 63, 768, 1), (500, 63, 640, 3), (64, 1000, 512, 2), (5, 5, 1024, 5)])
def test_skipped_entries_stay_untouched_when_k_is_long(mods, m, n, k, batch):
    """Plain-store products with few output tiles and a long k range are cut along k into slices that a second launch
    adds up.  With skip flags that second launch would write sums of slices nobody computed into the entries that are
    to be left alone, so such products are not cut."""
    _, X = mods
    g = torch.Generator().manual_seed(m + n + k)
    A, B = torch.randn(batch, m, k, generator=g).cuda(), torch.randn(batch, k, n, generator=g).cuda()
    want = (A.double() @ B.double()).cpu()
    for pipe in ("f32", "split"):
        for pattern in (0, 1):
            skip = torch.tensor([(b + pattern) % 2 for b in range(batch)], dtype=torch.int32).cuda()
            out = torch.full((batch, m, n), 7.0, device="cuda")
            X.gemm(A, B, out=out, skip=skip, pipe=pipe)
            for b in range(batch):
                if int(skip[b]):
                    assert bool((out[b] == 7.0).all()), (pipe, b)
                else:
                    assert rel_err(out[b], want[b]) <= TOL, (pipe, b)
