"""The stateful holders of qtensor.utils on the GPU (the callers of the boundary), checked against the
quantizer oracle, and the eigenbasis variant of the preconditioner (shampoo2) in low-bit mode."""
import numpy as np
import pytest
import torch

from oracle import quant_np as Q

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def U():
    import qtensor.functional as F
    import qtensor.utils as utils
    assert torch.cuda.is_available() and F.lib is not None
    return utils


def qmap(code_maps):
    return {"linear-2": torch.from_numpy(code_maps[("linear-2", 4)])}


def test_qtensor_and_diagreal_round_trip_and_buffer_reuse(U, code_maps):
    code = code_maps[("linear-2", 4)]
    g = torch.Generator().manual_seed(0)
    A = torch.randn(128, 128, generator=g)
    B = torch.randn(128, 128, generator=g)
    C = torch.randn(192, 192, generator=g)
    for cls, diag in ((U.QTensor, False), (U.QTensorDiagReal, True)):
        h = cls(A.cuda(), bits=4, name2qmap=qmap(code_maps), code="linear-2", blocksize=64, min_lowbit_size=4096)
        assert h.bits == 4 and h.var.dtype == torch.uint8 and h.var.numel() == 128 * 128 // 2
        assert h.name2qmap["linear-2"].is_cuda
        o = Q.quantize_c(A.numpy(), code, 128, 64, 4, diag)
        assert np.array_equal(h.var.cpu().numpy(), o[0]) and np.array_equal(h.absmax.cpu().numpy(), o[1])
        want = Q.dequantize_c(o[0], code, 128, o[1], 64, 4, diag=o[2] if diag else None)
        back = h.dequantize()
        assert back is not None and np.array_equal(back.cpu().numpy(), want)
        ptrs = (h.var.data_ptr(), h.absmax.data_ptr())
        h.quantize(B.cuda())                                   # same order: buffers are reused
        assert (h.var.data_ptr(), h.absmax.data_ptr()) == ptrs
        assert np.array_equal(h.var.cpu().numpy(), Q.quantize_c(B.numpy(), code, 128, 64, 4, diag)[0])
        h.quantize(C.cuda())                                   # another order: buffers are reallocated
        assert h.var_order == 192 and h.var.numel() == 192 * 192 // 2
        o = Q.quantize_c(C.numpy(), code, 192, 64, 4, diag)
        assert np.array_equal(h.var.cpu().numpy(), o[0])
        assert np.array_equal(h.dequantize().cpu().numpy(),
                              Q.dequantize_c(o[0], code, 192, o[1], 64, 4, diag=o[2] if diag else None))
        h.set_device("cuda")
        small = cls(torch.randn(32, 32).cuda(), bits=4, name2qmap=qmap(code_maps), code="linear-2", blocksize=64)
        assert small.bits == 32                                 # fewer than min_lowbit_size elements: dense
        h16 = cls(A.cuda().bfloat16(), bits=8, name2qmap={"linear-2": torch.from_numpy(code_maps[("linear-2", 8)])},
                  code="linear-2", blocksize=256, min_lowbit_size=4096)
        assert h16.dequantize().dtype == torch.bfloat16


def test_svdfast_low_bit_tracks_dense_eigenbasis(U, code_maps, tmp_path, monkeypatch):
    monkeypatch.chdir(tmp_path)
    g = torch.Generator().manual_seed(1)
    n = 128
    X_ = torch.randn(n, 4 * n, generator=g)
    L = (X_ @ X_.T / (4 * n)).cuda()
    kw = dict(name2qmap=qmap(code_maps), code="linear-2", blocksize=64, min_lowbit_size=4096)
    low = U.QTensorSVDFast(1e-6 * torch.eye(n, device="cuda"), bits=4, log_prefix="t_low", **kw)
    dense = U.QTensorSVDFast(1e-6 * torch.eye(n, device="cuda"), bits=32)
    assert low.bits == 4 and low.var.dtype == torch.uint8
    # the stored basis is exactly the quantized identity
    o = Q.quantize_c(np.eye(n, dtype=np.float32), code_maps[("linear-2", 4)], n, 64, 4)
    assert np.array_equal(low.var.cpu().numpy(), o[0])
    for _ in range(3):                                          # a few subspace-iteration updates
        for h in (low, dense):
            approx, vt = h.dequantize()
            h.quantize(0.9 * approx + 0.1 * L, vt)
    assert (tmp_path / "logs" / "eigenvalues_t_low.csv").is_file()
    a_low, vt_low = low.dequantize()
    a_dense, _ = dense.dequantize()
    assert float((vt_low @ vt_low.T - torch.eye(n, device="cuda")).abs().max()) < 0.05   # one Bjorck step after 4-bit storage
    assert float((a_low - a_dense).norm() / a_dense.norm()) < 0.5   # 4-bit storage error of the method itself
    assert float((low.Svalue - dense.Svalue).abs().max() / dense.Svalue.abs().max()) < 0.5
    p_low, p_dense = low.computepower(4, 1e-6), dense.computepower(4, 1e-6)
    assert p_low.shape == (n, n) and torch.isfinite(p_low).all()
    assert float((p_low - p_dense).norm() / p_dense.norm()) < 0.7


def test_svdfast_low_bit_follows_the_oracle_holder(U, code_maps, tmp_path, monkeypatch):
    """QTensorSVDFast in 4 bits against the CPU restatement of the reference holder (oracle/shampoo2_ref.py,
    R made positive on its diagonal), update by update from the same stored bits: codes, segment maxima,
    kept quotients and rows, largest quotient, rebuilt statistic and the inverse root from the eigenpairs."""
    from oracle.shampoo2_ref import RefEigenSlot
    monkeypatch.chdir(tmp_path)
    code = code_maps[("linear-2", 4)]
    g = torch.Generator().manual_seed(1)
    n = 128
    low = U.QTensorSVDFast(1e-6 * torch.eye(n, device="cuda"), bits=4, name2qmap=qmap(code_maps), code="linear-2",
                           blocksize=64, min_lowbit_size=4096)
    ref = RefEigenSlot(n, 1e-6, 4, code, 64, 4096, positive_r=True)
    flips = 0
    for _ in range(3):
        X_ = torch.randn(n, 4 * n, generator=g)
        L = X_ @ X_.T / (4 * n)
        codes, absmax = ref.codes()
        low.var.copy_(torch.from_numpy(codes)), low.absmax.copy_(torch.from_numpy(absmax))
        low.Svalue, low.keep_indices, low.max_eigenvalue = ref.svalue.cuda(), ref.keep.cuda(), ref.max_eig.cuda()
        a_ref, vt_ref = ref.dequantize()
        a_low, vt_low = low.dequantize()
        assert float((a_low.cpu() - a_ref).norm()) <= 1e-5 * max(float(a_ref.norm()), 1e-6)     # same bits in: rounding only
        assert float((vt_low.cpu() - vt_ref).abs().max()) <= 1e-5
        ref.quantize(0.9 * a_ref + 0.1 * L, vt_ref)
        low.quantize(0.9 * a_low + 0.1 * L.cuda(), vt_low)
        codes, absmax = ref.codes()
        got = low.var.cpu().numpy()
        flips += int(np.count_nonzero((got >> 4) != (codes >> 4)) + np.count_nonzero((got & 15) != (codes & 15)))
        assert float((low.absmax.cpu() - torch.from_numpy(absmax)).abs().max()) <= 1e-5 * float(absmax.max())
        assert torch.equal(low.keep_indices.cpu(), ref.keep)
        top = float(ref.max_eig)
        assert float((low.Svalue.cpu() - ref.svalue).abs().max()) <= 1e-5 * top
        assert abs(float(low.max_eigenvalue) - top) <= 1e-5 * top
        p_ref, p_low = ref.computepower(4, 1e-6), low.computepower(4, 1e-6).cpu()
        assert float((p_low - p_ref).norm() / p_ref.norm()) <= 5e-3                 # (a differing code or two)
    print("QTensorSVDFast: differing codes over three updates", flips, "of", 3 * n * n)
    assert flips <= 1e-3 * 3 * n * n


def test_shampoo2_low_bit_preconditioner_matches_host_recomputation_from_its_own_state(code_maps, tmp_path, monkeypatch):
    """4-bit eigenbasis storage is lossy by design, so the low-bit preconditioner is not compared with
    the 32-bit one; every stage is recomputed on the host from the state the holders actually store."""
    import qtensor.functional as F
    from optimizers import shampoo2 as S2
    from optimizers.matrix_functions import ComputePower
    monkeypatch.chdir(tmp_path)
    code = code_maps[("linear-2", 4)]
    g = torch.Generator().manual_seed(2)
    shape = (128, 192)
    kw = dict(stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=128, min_lowbit_size=4096, quan_blocksize=64)
    grads = [0.02 * torch.randn(shape, generator=g).cuda() for _ in range(3)]
    for mode in (0, 1):
        pre = S2.Preconditioner(torch.zeros(shape, device="cuda"), qmap(code_maps), prec_bits=4, inv_root_mode=mode, **kw)
        assert len(pre.statistics) == 4 and all(h.bits == 4 for h in pre.statistics + pre.preconditioners)
        for gr in grads:
            pre.add_statistics(gr)
        v0 = [torch.rand(h.var_order, generator=g) * 2 - 1 for h in pre.statistics]
        pre.compute_preconditioners(v0=[v.cuda() for v in v0])
        for h, prec, start in zip(pre.statistics, pre.preconditioners, v0):
            # the stored basis is a valid 4-bit state: it survives an oracle round trip unchanged
            n = h.var_order
            basis = torch.from_numpy(Q.dequantize_c(h.var.cpu().numpy(), code, n, h.absmax.cpu().numpy(), 64, 4))
            assert np.array_equal(h._basis().cpu().numpy(), basis.numpy())
            if mode == 0:
                want = F.compute_power(basis, h.Svalue.cpu(), 4, iter_count=4, ridge_epsilon=1e-6,
                                       indices=h.keep_indices.cpu(), max_eigen=h.max_eigenvalue.cpu())
            else:
                stat, _ = h.dequantize()
                want = ComputePower(stat.cpu(), 4, ridge_epsilon=1e-6, v0=start)
            o = Q.quantize_c(want.numpy(), code, n, 64, 4, True)
            want_q = torch.from_numpy(Q.dequantize_c(o[0], code, n, o[1], 64, 4, diag=o[2]))
            got_q = prec.dequantize().cpu()
            # matrix products differ in the last bits between host and device: segment maxima move by
            # an ulp and a code may flip at a tie
            far = (got_q - want_q).abs() > 1e-4 * want_q.abs().max()
            assert float(far.float().mean()) < 0.01
            assert float((got_q - want_q).norm() / want_q.norm()) < 0.02
        out = pre.preconditioned_grad(grads[-1])
        assert out.shape == shape and torch.isfinite(out).all()
        P = [p.dequantize().cpu().double() for p in pre.preconditioners]
        G = grads[-1].cpu().double()
        want = torch.cat([P[0] @ G[:, :128] @ P[1], P[2] @ G[:, 128:] @ P[3]], dim=1)
        assert float((out.cpu().double() - want).norm() / want.norm()) < 1e-5
