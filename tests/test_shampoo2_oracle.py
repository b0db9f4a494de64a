"""Pins for oracle/shampoo2_ref.py: run dense (32 bit) it must reproduce the reference's own
shampoo2 runs and its QTensorSVDFast bookkeeping; run low-bit it must be that same flow with the
(separately pinned) plain quantizer around the stored basis."""
import numpy as np
import torch

from oracle import quant_np as Q
from oracle.shampoo2_ref import RefEigenSlot, RefPreconditioner2, bjorck, orthonormal_factor


def rel(a, b):
    a, b = torch.as_tensor(a).double(), torch.as_tensor(b).double()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def start_vectors(seed, orders):
    torch.manual_seed(seed)                       # what the reference's global generator hands out
    return [torch.rand(o) * 2 - 1 for o in orders]


def test_dense_flow_reproduces_reference_runs_in_both_inverse_root_modes(golden):
    code = golden["linear2_4bit"]
    for tag, mode in (("s2m0", 0), ("s2m1", 1)):
        pre = RefPreconditioner2((6, 10), code, stat_decay=0.9, matrix_eps=1e-6, prec_maxorder=4, prec_bits=32,
                                 inv_root_mode=mode)
        orders = [s.order for s in pre.stats]
        assert np.array_equal(np.array([[o, o] for o in orders]), golden[f"pre_{tag}_shapes"])
        for st in range(3):
            grad = torch.from_numpy(golden[f"opt_grad_{st}_0"])
            pre.add_statistics(grad)
            pre.compute_preconditioners(start_vectors(1000 + st, orders))
            assert rel(pre.preconditioned_grad(grad), golden[f"pre_{tag}_out_{st}"]) <= 2e-5, (tag, st)
        for i, p in enumerate(pre.precs):
            assert rel(p.get(), golden[f"pre_{tag}_prec_{i}"]) <= 2e-5, (tag, i)


def test_eigenbasis_bookkeeping_reproduces_the_reference_holder(golden):
    n = 16
    slot = RefEigenSlot(n, 1e-6, 32, golden["linear2_4bit"], 64, 4096)
    approx0, vt0 = slot.dequantize()
    assert rel(approx0, golden["svd_init_dequant"]) <= 1e-6
    slot.quantize(torch.from_numpy(golden["svd_in"]), vt0)
    assert np.array_equal(slot.keep.numpy(), golden["svd_keep"])
    assert rel(slot.svalue, golden["svd_svalue"]) <= 1e-5
    assert abs(float(slot.max_eig) - float(golden["svd_maxeig"])) <= 1e-5 * float(golden["svd_maxeig"])
    assert rel(slot.basis(), golden["svd_vt"]) <= 1e-5          # rows are the eigenvector estimates (V^T, not V)
    assert rel(slot.dequantize()[0], golden["svd_dequant"]) <= 1e-5
    assert rel(slot.computepower(4, 1e-6), golden["svd_power"]) <= 1e-5
    # compute_power with Bjorck steps on a perturbed orthonormal basis
    slot.dense = torch.from_numpy(golden["cp_vt"]).clone()
    slot.keep = torch.from_numpy(golden["cp_keep"]).clone()
    slot.svalue = torch.from_numpy(golden["cp_s"]).clone()
    slot.max_eig = torch.tensor(3.0)
    assert rel(slot.computepower(4, 1e-6, steps=4), golden["cp_out"]) <= 1e-5
    assert rel(slot.computepower(4, 1e-6, steps=0), golden["cp_out"]) > 1e-4       # the steps matter


def test_bjorck_step_and_column_signs():
    g = torch.Generator().manual_seed(2)
    q, _ = torch.linalg.qr(torch.randn(24, 24, generator=g))
    rows = q[:10] + 0.02 * torch.randn(10, 24, generator=g)
    before = float((rows @ rows.T - torch.eye(10)).norm())
    after = float((bjorck(rows, 1) @ bjorck(rows, 1).T - torch.eye(10)).norm())
    assert after < 0.1 * before                                   # one step squares the defect (up to a constant)
    y = torch.randn(24, 24, generator=g)
    plain, fixed = orthonormal_factor(y), orthonormal_factor(y, positive_r=True)
    r = fixed.T @ y
    assert bool((torch.diagonal(r) > 0).all()) and float(torch.tril(r, -1).abs().max()) < 1e-5
    assert torch.equal(plain.abs(), fixed.abs())                  # only signs of whole columns differ
    assert float(((plain * fixed).sum(0).abs() - 1).abs().max()) < 1e-5


def test_low_bit_flow_is_the_dense_flow_through_the_plain_quantizer(golden):
    code = golden["linear2_4bit"]
    g = torch.Generator().manual_seed(4)
    grad = 0.02 * torch.randn(128, 192, generator=g)
    kw = dict(prec_maxorder=128, prec_bits=4, inv_root_mode=1, positive_r=True)
    low = RefPreconditioner2((128, 192), code, **kw)
    loop = RefPreconditioner2((128, 192), code, loop=True, **kw)
    assert [s.order for s in low.stats] == [128, 128, 128, 64] and all(s.low for s in low.stats)
    # the start is the quantized identity, read back exactly (1.0 is a table entry)
    assert torch.equal(low.stats[0].basis(), torch.eye(128))
    low.add_statistics(grad)
    loop.add_statistics(grad)
    # statistic 0 by hand: L = 0.95 * eps * diag(1 on the kept half) + 0.05 G G^T; QR of L I; V^T quantized plain
    blk = grad[:, :128]
    L = torch.zeros(128, 128)
    L[:64, :64] = 1e-6 * torch.eye(64)
    L.mul_(0.95).add_(blk @ blk.T, alpha=1 - 0.95)
    qf, rf = torch.linalg.qr(L)
    qf = qf * torch.sign(torch.diagonal(rf)).unsqueeze(0)
    want = Q.quantize_c(qf.T.contiguous().numpy(), code, 128, 64, 4, False)
    for got in (low.stats[0].codes(), tuple(x.numpy() for x in loop.stats[0].q)):
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    quot = (qf.T @ L @ qf).diag()
    assert rel(low.stats[0].svalue, torch.sort(quot)[0][:64]) <= 1e-5
    assert abs(float(low.stats[0].max_eig) - float(quot.max())) <= 1e-6 * float(quot.max())
    # the stored basis is 4-bit: the rebuilt statistic misses the larger half of the spectrum and the
    # re-encoding error, nothing else
    rebuilt, vt = low.stats[0].dequantize()
    assert float((vt @ vt.T - torch.eye(128)).abs().max()) < 0.2
    assert float(torch.linalg.eigvalsh(rebuilt.double())[-1]) <= 1.5 * float(low.stats[0].svalue.max())
    v0 = start_vectors(1, [128, 128, 128, 64])
    low.compute_preconditioners(v0)
    out = low.preconditioned_grad(grad)
    assert out.shape == grad.shape and torch.isfinite(out).all()
    # adopting a stored state reproduces the slot
    a, b = low.stats[1], RefEigenSlot(128, 1e-6, 4, code, 64, 4096, positive_r=True)
    b.load(*a.codes(), a.svalue, a.keep, a.max_eig)
    assert torch.equal(a.dequantize()[0], b.dequantize()[0])
    vec = RefPreconditioner2((5,), code)
    assert vec.preconditioned_grad(grad) is grad
