"""ctypes loader for the gfx950 quantization library (libqtensor_hip.so).

Same two entry points, return types and exception types as the reference loader
(qtensor/cextension.py:13-29 of the reference), but keyed on the ROCm build of torch:
the reference derives the file name from torch.version.cuda, which is None on
PyTorch-ROCm, so its loader can never find a library there.
"""
import ctypes as ct
import platform
from pathlib import Path

import torch

DYNAMIC_LIBRARY_SUFFIX = {"Linux": ".so"}.get(platform.system())
LIBRARY_STEM = "libqtensor_hip"


def get_cuda_version():
    """Digits of the GPU runtime version torch was built against ("70" for HIP 7.0.x).

    Kept under the reference's name; raises RuntimeError when torch has no GPU runtime
    at all (reference: qtensor/cextension.py:13-18)."""
    text = getattr(torch.version, "hip", None) or getattr(torch.version, "cuda", None)
    if not text:
        raise RuntimeError("This PyTorch build has neither a HIP nor a CUDA runtime.")
    major, minor = text.split(".")[:2]
    return f"{int(major)}{int(minor)}"


def library_path() -> Path:
    return (Path(__file__).parent / f"{LIBRARY_STEM}{DYNAMIC_LIBRARY_SUFFIX or '.so'}").resolve()


def get_lib():
    """Load libqtensor_hip.so from this directory (reference: qtensor/cextension.py:21-29).

    RuntimeError: torch is not a ROCm build, or the platform is not Linux.
    FileNotFoundError: the library has not been built (run csrc/build.sh)."""
    if not getattr(torch.version, "hip", None):
        raise RuntimeError("libqtensor_hip needs a ROCm build of PyTorch (torch.version.hip is empty).")
    get_cuda_version()
    if DYNAMIC_LIBRARY_SUFFIX is None:
        raise RuntimeError("The HIP quantization library is only built for Linux.")
    path = library_path()
    if not path.is_file():
        raise FileNotFoundError(f"Quantization library not found at {path}; build it with csrc/build.sh.")
    return ct.cdll.LoadLibrary(str(path))
