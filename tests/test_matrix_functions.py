"""matrix_functions on the CPU: reference vectors (seeded runs of the reference) and textbook identities."""
import numpy as np
import pytest
import torch

from optimizers.matrix_functions import ComputePower, MatPower, PowerIter, PowerIterBatched


def test_seeded_runs_reproduce_the_reference(golden):
    for tag in "abc":
        mat = torch.from_numpy(golden[f"newton_{tag}_in"])
        torch.manual_seed(7)
        lam, vec, iters = PowerIter(mat.clone())
        assert float(lam) == float(golden[f"poweriter_{tag}_lambda"])
        assert iters == int(golden[f"poweriter_{tag}_iters"])
        assert np.array_equal(vec.numpy(), golden[f"poweriter_{tag}_vec"])
        torch.manual_seed(7)
        root = ComputePower(mat.clone(), 4, ridge_epsilon=1e-6)
        want = torch.from_numpy(golden[f"newton_{tag}_out"])
        # same torch calls in the same order: bit-identical on the host that made the vectors,
        # and within GEMM rounding elsewhere
        assert torch.equal(root, want) or (root - want).norm() <= 1e-5 * want.norm()
    m = torch.from_numpy(golden["matpower_in"])
    assert torch.allclose(MatPower(m, 4), torch.from_numpy(golden["matpower_p4"]), rtol=1e-6, atol=1e-9)
    assert torch.allclose(MatPower(m, 3), torch.from_numpy(golden["matpower_p3"]), rtol=1e-6, atol=1e-9)
    assert np.allclose(ComputePower(torch.tensor([1.0, 4.0, 16.0]), 4).numpy(), golden["newton_vector_out"])
    assert np.array_equal(ComputePower(torch.tensor([[5.0]]), 4).numpy(), golden["newton_1x1_out"])


def test_inverse_root_identity_on_well_conditioned_input():
    g = torch.Generator().manual_seed(0)
    n = 40
    q, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
    lam = torch.linspace(0.5, 2.0, n, dtype=torch.float64)
    G = ((q * lam) @ q.T).float()
    v0 = torch.rand(n, generator=g) * 2 - 1
    arg = G.clone()
    root = ComputePower(arg, 4, ridge_epsilon=1e-6, v0=v0)
    ridge = (arg - G).diagonal().mean().double()                 # the in-place ridge that was added
    assert 1e-6 * 1.0 < ridge < 1e-6 * 2.1
    exact = (q * (lam + ridge) ** -0.25) @ q.T
    assert (root.double() - exact).norm() / exact.norm() < 1e-5
    r4 = MatPower(root.double(), 4)
    assert (r4 @ (G.double() + ridge * torch.eye(n)) - torch.eye(n)).abs().max() < 1e-4


def test_matpower_against_repeated_products():
    g = torch.Generator().manual_seed(1)
    m = torch.randn(6, 6, generator=g, dtype=torch.float64) / 3
    for p in (1, 2, 3, 4, 5, 7, 8, 11, 16):
        want = torch.eye(6, dtype=torch.float64)
        for _ in range(p):
            want = want @ m
        assert torch.allclose(MatPower(m, p), want, rtol=1e-10, atol=1e-12)


def test_power_iteration_forms_agree_and_stop_early():
    g = torch.Generator().manual_seed(2)
    mats = []
    for n_big in (1.0, 50.0, 3.0):
        q, _ = torch.linalg.qr(torch.randn(24, 24, generator=g))
        lam = torch.linspace(0.01, 1.0, 24)
        lam[-1] = n_big                                          # dominant eigenvalue: fast convergence when large
        mats.append((q * lam) @ q.T)
    stack = torch.stack(mats)
    v0 = torch.rand(3, 24, generator=g) * 2 - 1
    batched = PowerIterBatched(stack, v0=v0)
    for b in range(3):
        single, _, iters = PowerIter(stack[b], v0=v0[b])
        assert abs(float(batched[b]) - float(single)) <= 2e-6 * abs(float(single))
    _, _, iters = PowerIter(stack[1], v0=v0[1])
    assert iters < 10                                            # converged before the cap
