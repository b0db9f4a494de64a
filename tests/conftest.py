import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
PKG = ROOT / "low-bit-shampoo_amd"
for p in (str(ROOT), str(PKG)):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    with np.load(ROOT / "tests" / "golden" / "reference_vectors.npz") as z:
        return {k: z[k] for k in z.files}


@pytest.fixture(scope="session")
def code_maps(golden):
    return {
        ("linear-2", 4): golden["linear2_4bit"],
        ("linear-2", 8): golden["linear2_8bit"],
        ("dynamic", 4): golden["dynamic_4bit"],
        ("dynamic", 8): golden["dynamic_8bit"],
    }
