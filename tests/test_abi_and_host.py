"""CPU-side checks: the C-ABI library loads and exports every declared symbol, and the host
mirror of qtensor behaves like the reference's interface where no GPU is involved."""
import ctypes as ct
import re
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "qtensor_hip.h"
LIB = ROOT / "low-bit-shampoo_amd" / "qtensor" / "libqtensor_hip.so"

REFERENCE_SYMBOLS = [f"c{kind}_blockwise{mid}_{bits}bit_{dt}"
                     for kind in ("quantize", "dequantize") for mid in ("", "_diagreal")
                     for bits in (8, 4) for dt in ("fp32", "bf16")]


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", " ".join(
        line for line in text.splitlines() if not line.lstrip().startswith("#") and "typedef" not in line))))


@pytest.fixture(scope="module")
def built_library():
    if not LIB.is_file():
        subprocess.run(["bash", str(ROOT / "low-bit-shampoo_amd" / "csrc" / "build.sh")], check=True)
    return LIB


def test_header_declares_the_sixteen_reference_entry_points():
    names = declared_functions()
    assert len(REFERENCE_SYMBOLS) == 16
    for sym in REFERENCE_SYMBOLS:
        assert sym in names and sym + "_stream" in names


def test_library_loads_and_exports_every_declared_symbol(built_library):
    lib = ct.CDLL(str(built_library))
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in qtensor_hip.h but not exported"
    lib.qtensor_hip_version.restype = ct.c_int
    assert lib.qtensor_hip_version() >= 100
    exported = subprocess.run(["nm", "-D", "--defined-only", str(built_library)], capture_output=True, text=True,
                              check=True).stdout
    for sym in REFERENCE_SYMBOLS:
        assert re.search(rf"\bT {sym}\b", exported)


def test_loader_keeps_reference_names_and_exception_types(monkeypatch, built_library):
    import qtensor.cextension as cx
    assert cx.get_cuda_version().isdigit()
    assert isinstance(cx.get_lib(), ct.CDLL)
    monkeypatch.setattr(cx, "LIBRARY_STEM", "libqtensor_not_built")
    with pytest.raises(FileNotFoundError):
        cx.get_lib()
    monkeypatch.setattr(cx.torch.version, "hip", None)
    with pytest.raises(RuntimeError):
        cx.get_lib()
    monkeypatch.setattr(cx.torch.version, "cuda", None, raising=False)
    with pytest.raises(RuntimeError):
        cx.get_cuda_version()


def test_functional_surface_and_no_cpu_fallback(built_library):
    import qtensor.functional as F
    for name in ("quantize_blockwise", "dequantize_blockwise", "quantize_blockwise_diagreal",
                 "dequantize_blockwise_diagreal", "create_dynamic_map", "create_linear_map", "get_ptr",
                 "compute_power", "lib", "lib_quan", "lib_dequan", "lib_quan_diagreal", "lib_dequan_diagreal"):
        assert hasattr(F, name)
    assert F.lib is not None and set(F.lib_quan) == {4, 8} and len(F.lib_dequan_diagreal[4]) == 2
    assert F.get_ptr(None) is None
    t = torch.zeros(4)
    assert F.get_ptr(t).value == t.data_ptr()
    code = F.create_linear_map(True, 4, 2)
    A = torch.randn(64, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        F.quantize_blockwise(A, code, 64, blocksize=64, bits=4)
    with pytest.raises(RuntimeError, match="GPU only"):
        F.dequantize_blockwise(torch.zeros(2048, dtype=torch.uint8), code, 64, torch.zeros(64), blocksize=64, bits=4)
    with pytest.raises(RuntimeError, match="GPU only"):
        F.quantize_blockwise_diagreal(A, code, 64, blocksize=64, bits=4)


def test_code_map_builders_reproduce_the_reference_bits(code_maps):
    import qtensor.functional as F
    for (name, bits), want in code_maps.items():
        got = (F.create_linear_map(True, bits, 2) if name == "linear-2" else F.create_dynamic_map(True, bits, 1)).numpy()
        # identical torch calls on the same host give identical bits; another host's vector
        # width may move single entries by an ulp (torch.linspace), never more
        assert got.shape == want.shape
        assert np.array_equal(got, want) or np.max(np.abs(got.view(np.int32).astype(np.int64) -
                                                          want.view(np.int32).astype(np.int64))) <= 4
    u = F.create_linear_map(False, 4, 2)
    assert u[0] == 0 and u[-1] == 1 and torch.all(u[1:] > u[:-1])
    d = F.create_dynamic_map(False, 8, 1)
    assert d.numel() == 256 and d.min() == 0 and d.max() == 1


def test_compute_power_matches_reference_vectors(golden):
    import qtensor.functional as F
    out = F.compute_power(torch.from_numpy(golden["cp_vt"]), torch.from_numpy(golden["cp_s"]), 4, iter_count=4,
                          ridge_epsilon=1e-6, indices=torch.from_numpy(golden["cp_keep"]),
                          max_eigen=torch.tensor(3.0))
    assert torch.allclose(out, torch.from_numpy(golden["cp_out"]), rtol=1e-5, atol=1e-6)
    # closed form: for exactly orthonormal rows the result is V^T diag((s+rho)^-1/4) V
    q, _ = torch.linalg.qr(torch.randn(8, 8, dtype=torch.float64))
    s = torch.linspace(0.5, 2, 8, dtype=torch.float64)
    got = F.compute_power(q.T.contiguous(), s, 4, iter_count=2, ridge_epsilon=0.0)
    assert torch.allclose(got, q @ torch.diag(s ** -0.25) @ q.T, atol=1e-12)


def test_dense_holders_need_no_gpu():
    from qtensor.utils import QTensor, QTensorDiagReal, QTensorSVDFast
    M = torch.randn(8, 8)
    for cls in (QTensor, QTensorDiagReal):
        h = cls(M, bits=32)
        assert h.bits == 32 and torch.equal(h.dequantize(), M)
        h.quantize(2 * M)
        assert torch.equal(h.dequantize(), 2 * M)
        h16 = cls(M, bits=16)
        assert h16.bits == 16 and h16.dequantize().dtype == torch.bfloat16
        small = cls(M, bits=4, name2qmap={"linear-2": torch.zeros(16)}, code="linear-2", min_lowbit_size=4096)
        assert small.bits == 32                                # too small to quantize: stays dense
    with pytest.raises(ValueError):
        QTensor(torch.randn(64, 64), bits=5, min_lowbit_size=16)
    s = QTensorSVDFast(1e-6 * torch.eye(8), bits=32)
    approx, vt = s.dequantize()
    assert torch.equal(vt, torch.eye(8)) and approx.shape == (8, 8)


def test_svdfast_dense_path_matches_reference_vectors(golden):
    from qtensor.utils import QTensorSVDFast
    n = golden["svd_in"].shape[0]
    s = QTensorSVDFast(1e-6 * torch.eye(n), bits=32)
    approx0, vt0 = s.dequantize()
    assert torch.allclose(approx0, torch.from_numpy(golden["svd_init_dequant"]))
    s.quantize(torch.from_numpy(golden["svd_in"]), vt0)
    assert torch.equal(s.keep_indices, torch.from_numpy(golden["svd_keep"]))
    assert torch.allclose(s.Svalue, torch.from_numpy(golden["svd_svalue"]), rtol=1e-5, atol=1e-7)
    assert abs(float(s.max_eigenvalue) - float(golden["svd_maxeig"])) <= 1e-5 * float(golden["svd_maxeig"])
    approx1, _ = s.dequantize()
    assert torch.allclose(approx1, torch.from_numpy(golden["svd_dequant"]), rtol=1e-4, atol=1e-6)
    assert torch.allclose(s.computepower(4, ridge_epsilon=1e-6), torch.from_numpy(golden["svd_power"]),
                          rtol=1e-4, atol=1e-5)
    # invariants: Rayleigh quotients of an orthonormal basis lie inside the spectrum, the kept
    # ones are the smaller half, and the basis rows are orthonormal
    lam = torch.linalg.eigvalsh(torch.from_numpy(golden["svd_in"]).double())
    assert float(s.Svalue.min()) >= float(lam[0]) - 1e-5 and float(s.max_eigenvalue) <= float(lam[-1]) + 1e-5
    assert float(s.Svalue.max()) <= float(s.max_eigenvalue) and s.Svalue.numel() == n // 2
    assert torch.allclose(s.var @ s.var.T, torch.eye(n), atol=1e-5)


def test_bench_refuses_more_than_one_gpu_and_names_its_sections():
    """bench.py measures one GPU: --gpus N with N > 1 exits with a message (no GPU is touched for that)."""
    bench = ROOT / "bench.py"
    run = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0 and "one GPU" in (run.stderr + run.stdout)
    helptext = subprocess.run([sys.executable, str(bench), "--help"], capture_output=True, text=True, check=True).stdout
    for flag in ("--gpus", "--steps", "--warmup", "--section", "--no-cpu-baseline"):
        assert flag in helptext
