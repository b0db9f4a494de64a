"""Writes tests/golden/reference_vectors.npz by running a few reference functions.

Run in the build container only (the reference checkout is not available anywhere
else):  python tests/golden/make_reference_vectors.py [/root/reference]

Only functions whose exact outputs nothing else pins are executed here:
  * the code-map builders (their bits come from torch.linspace's CPU kernel, which
    depends on the host's vector width, plus a float64 scaling step),
  * the seeded coupled-Newton inverse root and power iteration (they draw from the
    global torch RNG),
  * the eigenbasis bookkeeping of the 32-bit QTensorSVDFast path (QR signs, sort order),
  * compute_power (Bjorck steps + inverse root in the kept subspace),
  * the preconditioner / optimizer step logic of optimizers/shampoo1.py and shampoo2.py on tiny
    CPU parameters (block partitioning, statistics update, inverse roots, grafting, SGD and
    AdamW updates).
The blockwise quantizer itself is not run: IEEE-754 plus the written rules fix it.
The reference's prebuilt native libraries are never loaded (its loader raises on a
build of torch without a CUDA version string before it touches any file).
"""
import sys
from pathlib import Path

import numpy as np
import torch


def optimizer_runs():
    """A few steps of the reference's preconditioners and optimizers on tiny CPU parameters (the
    reference keeps everything in 32 bit on the CPU).  The global generator is re-seeded before
    every step because the power iteration draws its start vector from it."""
    import os
    import tempfile

    from optimizers import shampoo1 as R1
    from optimizers import shampoo2 as R2

    res = {}
    cwd = os.getcwd()
    with tempfile.TemporaryDirectory() as tmp:
        os.chdir(tmp)                                   # shampoo2 writes logs/*.csv on first use
        try:
            g = torch.Generator().manual_seed(42)
            shapes = [(6, 10), (5,), (4, 1, 3), (9, 9)]
            grads = [[torch.randn(s, generator=g) for s in shapes] for _ in range(4)]
            init = [torch.randn(s, generator=g) for s in shapes]
            for k, t in enumerate(init):
                res[f"opt_init_{k}"] = t.numpy().copy()
            for st, gs in enumerate(grads):
                for k, t in enumerate(gs):
                    res[f"opt_grad_{st}_{k}"] = t.numpy().copy()

            # bare preconditioners
            for tag, mod, kw in (("s1", R1, {}), ("s2m0", R2, dict(inv_root_mode=0)), ("s2m1", R2, dict(inv_root_mode=1))):
                var = init[0].clone()
                pre = mod.Preconditioner(var, {}, stat_decay=0.9, matrix_eps=1e-6, prec_maxorder=4, prec_bits=32, **kw)
                res[f"pre_{tag}_shapes"] = np.array(pre._partitioner.shapes_for_preconditioners())
                for st in range(3):
                    torch.manual_seed(1000 + st)
                    pre.add_statistics(grads[st][0])
                    pre.compute_preconditioners()
                    res[f"pre_{tag}_out_{st}"] = pre.preconditioned_grad(grads[st][0]).numpy().copy()
                for i, h in enumerate(pre.preconditioners):
                    res[f"pre_{tag}_prec_{i}"] = h.dequantize().numpy().copy()
                if tag == "s1":
                    for i, h in enumerate(pre.statistics):
                        res[f"pre_{tag}_stat_{i}"] = h.dequantize().numpy().copy()

            # whole optimizers
            runs = (("adamw1", R1.ShampooAdamW, dict(lr=1e-2, weight_decay=0.05)),
                    ("sgd1", R1.ShampooSGD, dict(lr=1e-2, momentum=0.9, weight_decay=1e-3, nesterov=True)),
                    ("adamw2", R2.ShampooAdamW, dict(lr=1e-2, weight_decay=0.05, inv_root_mode=0)),
                    ("sgd2", R2.ShampooSGD, dict(lr=1e-2, momentum=0.9, inv_root_mode=1)))
            for tag, cls, kw in runs:
                params = [torch.nn.Parameter(t.clone()) for t in init]
                opt = cls(params, start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2, stat_decay=0.9,
                          prec_maxorder=4, prec_bits=32, **kw)
                for st in range(4):
                    for p_, g_ in zip(params, grads[st]):
                        p_.grad = g_.clone()
                    torch.manual_seed(2000 + st)
                    opt.step()
                for k, p_ in enumerate(params):
                    res[f"opt_{tag}_final_{k}"] = p_.detach().numpy().copy()
        finally:
            os.chdir(cwd)
    return res


def main() -> None:
    ref_root = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    sys.path.insert(0, str(ref_root))
    import qtensor.functional as RF  # noqa: E402
    from qtensor.utils import QTensorSVDFast  # noqa: E402
    from optimizers.matrix_functions import ComputePower, MatPower, PowerIter  # noqa: E402

    assert RF.lib is None, "reference native library must not be loaded"
    out = {}

    out["linear2_4bit"] = RF.create_linear_map(True, 4, 2).numpy()
    out["linear2_8bit"] = RF.create_linear_map(True, 8, 2).numpy()
    out["dynamic_8bit"] = RF.create_dynamic_map(True, 8, 1).numpy()
    out["dynamic_4bit"] = RF.create_dynamic_map(True, 4, 1).numpy()

    # Inverse 4th root by coupled Newton, on seeded PSD inputs (float32, CPU).
    for tag, n, cond in (("a", 12, 1e2), ("b", 32, 1e4), ("c", 48, 1e6)):
        g = torch.Generator().manual_seed(100 + n)
        q, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
        lam = torch.logspace(0, -float(np.log10(cond)), n, dtype=torch.float64)
        mat = (q * lam) @ q.T
        mat = ((mat + mat.T) / 2).float()
        out[f"newton_{tag}_in"] = mat.numpy().copy()
        torch.manual_seed(7)
        lam_max, vec, iters = PowerIter(mat.clone())
        out[f"poweriter_{tag}_lambda"] = np.float32(lam_max.item())
        out[f"poweriter_{tag}_vec"] = vec.numpy().copy()
        out[f"poweriter_{tag}_iters"] = np.int64(iters)
        torch.manual_seed(7)
        root = ComputePower(mat.clone(), 4, ridge_epsilon=1e-6)
        out[f"newton_{tag}_out"] = root.numpy().copy()
    out["matpower_in"] = out["newton_a_in"] * np.float32(0.5)
    out["matpower_p4"] = MatPower(torch.from_numpy(out["matpower_in"]), 4).numpy()
    out["matpower_p3"] = MatPower(torch.from_numpy(out["matpower_in"]), 3).numpy()
    out["newton_vector_out"] = ComputePower(torch.tensor([1.0, 4.0, 16.0]), 4).numpy()
    out["newton_1x1_out"] = ComputePower(torch.tensor([[5.0]]), 4).numpy()

    # Eigenbasis statistic held in 32 bit: update with a new matrix, then read back.
    n = 16
    g = torch.Generator().manual_seed(5)
    a = torch.randn(n, 3 * n, generator=g)
    stat0 = a @ a.T / (3 * n)
    qt = QTensorSVDFast(1e-6 * torch.eye(n), bits=32)
    approx0, vt0 = qt.dequantize()
    out["svd_init_dequant"] = approx0.numpy().copy()
    qt.quantize(stat0, vt0)
    out["svd_in"] = stat0.numpy().copy()
    out["svd_keep"] = qt.keep_indices.numpy().copy()
    out["svd_svalue"] = qt.Svalue.numpy().copy()
    out["svd_maxeig"] = np.float32(qt.max_eigenvalue.item())
    out["svd_vt"] = qt.var.numpy().copy()
    approx1, _ = qt.dequantize()
    out["svd_dequant"] = approx1.numpy().copy()
    out["svd_power"] = qt.computepower(4, ridge_epsilon=1e-6).numpy().copy()

    # compute_power with Bjorck steps on a slightly perturbed orthonormal basis.
    g = torch.Generator().manual_seed(11)
    qmat, _ = torch.linalg.qr(torch.randn(n, n, generator=g))
    vt = (qmat.T + 1e-3 * torch.randn(n, n, generator=g)).contiguous()
    s = torch.linspace(0.1, 2.0, n // 2)
    keep = torch.arange(0, n, 2)
    out["cp_vt"] = vt.numpy().copy()
    out["cp_s"] = s.numpy().copy()
    out["cp_keep"] = keep.numpy().copy()
    out["cp_out"] = RF.compute_power(vt, s, 4, iter_count=4, ridge_epsilon=1e-6,
                                     indices=keep, max_eigen=torch.tensor(3.0)).numpy().copy()

    out.update(optimizer_runs())

    dest = Path(__file__).with_name("reference_vectors.npz")
    np.savez_compressed(dest, **out)
    print(f"wrote {dest} with {len(out)} arrays; torch {torch.__version__}, "
          f"cpu capability {torch.backends.cpu.get_cpu_capability()}")


if __name__ == "__main__":
    main()
