"""Pins for oracle/shampoo_ref.py: run dense (32 bit) it must reproduce the reference's own runs;
run low-bit it must be that same dense flow with the quantizer oracle in between."""
import numpy as np
import torch

from oracle import quant_np as Q
from oracle.shampoo_ref import RefPreconditioner, newton_root, pieces


def rel(a, b):
    a, b = torch.as_tensor(a).double(), torch.as_tensor(b).double()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def start_vectors(seed, orders):
    torch.manual_seed(seed)                       # what the reference's global generator hands out
    return [torch.rand(o) * 2 - 1 for o in orders]


def test_dense_flow_reproduces_reference_runs(golden):
    code = golden["linear2_4bit"]
    pre = RefPreconditioner((6, 10), code, stat_decay=0.9, matrix_eps=1e-6, prec_maxorder=4, prec_bits=32)
    orders = [s.order for s in pre.stats]
    assert np.array_equal(np.array([[o, o] for o in orders]), golden["pre_s1_shapes"])
    for st in range(3):
        grad = torch.from_numpy(golden[f"opt_grad_{st}_0"])
        pre.add_statistics(grad)
        pre.compute_preconditioners(start_vectors(1000 + st, orders))
        assert rel(pre.preconditioned_grad(grad), golden[f"pre_s1_out_{st}"]) <= 2e-5
    for i, (s, p) in enumerate(zip(pre.stats, pre.precs)):
        assert rel(s.get(), golden[f"pre_s1_stat_{i}"]) <= 2e-5
        assert rel(p.get(), golden[f"pre_s1_prec_{i}"]) <= 2e-5


def test_newton_restatement_reproduces_reference_vectors(golden):
    for tag in "abc":
        mat = torch.from_numpy(golden[f"newton_{tag}_in"]).clone()
        torch.manual_seed(7)
        v0 = torch.rand(mat.shape[0]) * 2 - 1
        assert rel(newton_root(mat, 4, 1e-6, v0), golden[f"newton_{tag}_out"]) <= 1e-5
    assert pieces(2304, 1024) == [1024, 1024, 256] and pieces(1024, 1024) == [1024] and pieces(7, 0) == [7]


def test_low_bit_flow_is_the_dense_flow_through_the_quantizer(golden):
    code = golden["linear2_4bit"]
    g = torch.Generator().manual_seed(4)
    grad = 0.02 * torch.randn(128, 192, generator=g)
    low = RefPreconditioner((128, 192), code, prec_maxorder=128, prec_bits=4)
    loop = RefPreconditioner((128, 192), code, prec_maxorder=128, prec_bits=4, loop=True)
    assert [s.order for s in low.stats] == [128, 128, 128, 64]
    assert [s.low for s in low.stats] == [True, True, True, True]
    low.add_statistics(grad)
    loop.add_statistics(grad)
    # statistic 0 by hand: quantize(eps I) -> dequantize -> decay + Gram -> quantize
    q0 = Q.quantize_c((1e-6 * torch.eye(128)).numpy(), code, 128, 64, 4, True)
    cur = torch.from_numpy(Q.dequantize_c(q0[0], code, 128, q0[1], 64, 4, diag=q0[2]).copy())
    blk = grad[:, :128]
    cur.mul_(0.95).add_(blk @ blk.T, alpha=1 - 0.95)
    want = Q.quantize_c(cur.numpy(), code, 128, 64, 4, True)
    for got in (low.stats[0].codes(), loop.stats[0].codes()):
        for a, b in zip(got, want):
            assert np.array_equal(a, b)
    v0 = start_vectors(1, [128, 128, 128, 64])
    low.compute_preconditioners(v0)
    out = low.preconditioned_grad(grad)
    assert out.shape == grad.shape and torch.isfinite(out).all()
    # a vector parameter is passed through untouched
    vec = RefPreconditioner((5,), code)
    assert vec.preconditioned_grad(grad) is grad
