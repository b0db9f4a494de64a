"""Writes tests/golden/reference_vectors.npz by running a few reference functions.

Run in the build container only (the reference checkout is not available anywhere
else):  python tests/golden/make_reference_vectors.py [/root/reference]

Only functions whose exact outputs nothing else pins are executed here:
  * the code-map builders (their bits come from torch.linspace's CPU kernel, which
    depends on the host's vector width, plus a float64 scaling step),
  * the seeded coupled-Newton inverse root and power iteration (they draw from the
    global torch RNG),
  * the eigenbasis bookkeeping of the 32-bit QTensorSVDFast path (QR signs, sort order),
  * compute_power (Bjorck steps + inverse root in the kept subspace).
The blockwise quantizer itself is not run: IEEE-754 plus the written rules fix it.
The reference's prebuilt native libraries are never loaded (its loader raises on a
build of torch without a CUDA version string before it touches any file).
"""
import sys
from pathlib import Path

import numpy as np
import torch


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

    dest = Path(__file__).with_name("reference_vectors.npz")
    np.savez_compressed(dest, **out)
    print(f"wrote {dest} with {len(out)} arrays; torch {torch.__version__}, "
          f"cpu capability {torch.backends.cpu.get_cpu_capability()}")


if __name__ == "__main__":
    main()
