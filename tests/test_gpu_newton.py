"""GPU parity of the batched coupled-Newton inverse root against the CPU restatement of the reference's
algorithm (oracle/shampoo_ref.py: power_iteration, newton_root; reference optimizers/matrix_functions.py:21-141,
pinned to the reference's own seeded runs in tests/test_shampoo_oracle.py) with the same start vectors."""
import pytest
import torch

from optimizers.matrix_functions import ComputePowerBatched, PowerIterBatched
from oracle.shampoo_ref import newton_root, power_iteration

pytestmark = pytest.mark.gpu


def ComputePower(mat, p, ridge_epsilon, v0):
    return newton_root(mat, p, ridge_epsilon, v0)


def PowerIter(mat, v0):
    return power_iteration(mat, v0), None, None


def psd_stack(batch, n, cond, seed):
    g = torch.Generator().manual_seed(seed)
    mats = []
    for _ in range(batch):
        q, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
        lam = 10.0 ** (-cond * torch.rand(n, generator=g, dtype=torch.float64))
        m = (q * lam) @ q.T
        mats.append(((m + m.T) / 2).float())
    return torch.stack(mats), torch.rand(batch, n, generator=g) * 2 - 1


@pytest.mark.parametrize("n,batch,cond", [(64, 5, 1.0), (256, 3, 2.0), (768, 2, 3.0), (100, 4, 2.0), (1024, 1, 4.0)])
def test_batched_newton_matches_cpu_iteration(n, batch, cond):
    mats, v0 = psd_stack(batch, n, cond, seed=n)
    got = ComputePowerBatched(mats.clone().cuda(), 4, ridge_epsilon=1e-6, v0=v0).cpu()
    for b in range(batch):
        want = ComputePower(mats[b].clone(), 4, ridge_epsilon=1e-6, v0=v0[b])
        rel = float((got[b] - want).norm() / want.norm())
        # same iteration, same start vector; only the rounding inside the fp32 products differs.
        # The iteration damps such perturbations for well-conditioned input; the bound grows with
        # the condition number of the problem (measured: 1e-6 .. 3e-5 over these cases).
        assert rel <= (1e-5 if cond <= 2.0 else 1e-4), (n, b, rel)
        # and against the definition in float64 for the well-conditioned cases
        if cond <= 2.0:
            lam, vec = torch.linalg.eigh(mats[b].double())
            top, _, _ = PowerIter(mats[b], v0=v0[b])
            exact = (vec * (lam + 1e-6 * float(top)) ** -0.25) @ vec.T
            assert float((got[b].double() - exact).norm() / exact.norm()) <= 1e-4


def test_batched_power_iteration_and_stopping_rules():
    mats, v0 = psd_stack(4, 128, 1.0, seed=3)
    top = PowerIterBatched(mats.cuda(), v0=v0).cpu()
    for b in range(4):
        want, _, _ = PowerIter(mats[b], v0=v0[b])
        assert abs(float(top[b]) - float(want)) <= 1e-5 * float(want)
    # a matrix that is already the identity needs no round; one far from it needs them all
    eye = torch.eye(64)
    stack = torch.stack([eye * 1.0, torch.diag(torch.logspace(0, -5, 64))]).cuda()
    out = ComputePowerBatched(stack.clone(), 4, ridge_epsilon=0.0, v0=torch.ones(2, 64)).cpu()
    for b in range(2):
        want = ComputePower(stack[b].cpu().clone(), 4, ridge_epsilon=0.0, v0=torch.ones(64))
        assert float((out[b] - want).norm() / want.norm()) <= 1e-5
    one = ComputePowerBatched(torch.full((3, 1, 1), 5.0, device="cuda"), 4)
    assert torch.equal(one.cpu(), torch.ones(3, 1, 1))


@pytest.mark.parametrize("n,cond", [(768, 4.0), (768, 6.0), (1024, 4.0), (1024, 6.0), (256, 6.0)])
def test_ill_conditioned_inverse_roots_are_as_good_as_the_cpu_iteration(n, cond):
    """Eigenvalues log-uniform in [10^-cond, 1] (the spread of the statistics in the fused-product and ViT-B/32
    workloads).  Ten Newton rounds in fp32 do not reach the definition (G + r I)^(-1/4) to 1e-5 there, on any
    machine; the claim is that the matrix-core path is as close to it as the reference's own fp32 arithmetic on
    the CPU: error(GPU) <= 2 * error(CPU fp32 iteration) + 1e-5, both measured against float64 eigh, and the
    two fp32 results agree with each other to a small multiple of the CPU's own error."""
    batch = 2
    mats, v0 = psd_stack(batch, n, cond, seed=int(n + cond))
    got = ComputePowerBatched(mats.clone().cuda(), 4, ridge_epsilon=1e-6, v0=v0).cpu()
    for b in range(batch):
        cpu = ComputePower(mats[b].clone(), 4, ridge_epsilon=1e-6, v0=v0[b])
        lam, vec = torch.linalg.eigh(mats[b].double())
        top, _, _ = PowerIter(mats[b], v0=v0[b])
        exact = (vec * (lam + 1e-6 * float(top)) ** -0.25) @ vec.T
        e_cpu = float((cpu.double() - exact).norm() / exact.norm())
        e_gpu = float((got[b].double() - exact).norm() / exact.norm())
        apart = float((got[b] - cpu).norm() / cpu.norm())
        print(f"n {n} cond 1e{cond:.0f}: error of the CPU fp32 iteration {e_cpu:.2e}, of the GPU {e_gpu:.2e}, apart {apart:.2e}")
        assert e_gpu <= 2 * e_cpu + 1e-5, (n, cond, b, e_cpu, e_gpu)
        assert apart <= 5e-5, (n, cond, b, apart)


@pytest.mark.parametrize("n,batch", [(64, 3), (100, 2), (1024, 5), (1500, 1), (7, 4)])
def test_stack_matrix_vector_product(n, batch):
    """The library's matrix-vector product for a whole stack (the power iteration's only product) against float64."""
    import qtensor.fused as X
    g = torch.Generator().manual_seed(n)
    mats, v = torch.randn(batch, n, n, generator=g), torch.randn(batch, n, generator=g)
    got = X.matvec(mats.cuda(), v.cuda())
    want = torch.bmm(mats.double(), v.double().unsqueeze(2)).squeeze(2)
    scale = torch.bmm(mats.double().abs(), v.double().abs().unsqueeze(2)).squeeze(2)
    assert got.shape == (batch, n)
    assert float(((got.cpu().double() - want).abs() / scale).max()) <= 1e-6
    assert torch.equal(got, X.matvec(mats.cuda(), v.cuda()))                   # fixed summation order
    view = torch.zeros(batch, n, n + 4, device="cuda")[:, :, 1:n + 1]            # not contiguous: refused
    with pytest.raises(ValueError):
        X.matvec(view, v.cuda())
