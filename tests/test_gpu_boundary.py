"""The drop-in boundary exercised the way the reference exercises it: libqtensor_hip.so loaded with a bare
ctypes handle, NO argtypes, pointers as c_void_p(tensor.data_ptr()), integers as c_int32, the null stream
(reference: qtensor/functional.py:17-60 binds the sixteen symbols, :68-84 get_ptr, :145-155, :193-211,
:251-282, :325-343 call them).  All sixteen are called on the device -- 4 and 8 bit, fp32 and bf16, plain
and with the exact diagonal, quantize and dequantize -- and compared bit for bit with the C oracle."""
import ctypes as ct
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import quant_np as Q

pytestmark = pytest.mark.gpu
LIB = Path(__file__).resolve().parents[1] / "low-bit-shampoo_amd" / "qtensor" / "libqtensor_hip.so"


def get_ptr(t):
    return None if t is None else ct.c_void_p(t.data.data_ptr())


def bits_of(x):
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("order,blocksize", [(256, 64), (200, 128), (129, 64)])      # flat layout, ragged rows, odd order
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_sixteen_reference_symbols_bound_like_the_reference_binds_them(code_maps, order, blocksize, bits, dtype):
    assert torch.cuda.is_available()
    lib = ct.cdll.LoadLibrary(str(LIB))                    # what the reference's get_lib() returns
    code_np = code_maps[("linear-2", bits)]
    code = torch.from_numpy(code_np).cuda()
    g = torch.Generator().manual_seed(order * bits)
    A = torch.randn(order, order, generator=g)
    A[3, 3:40] = 0.0                                       # a zero stretch (a whole segment when blocksize is 64... or not)
    A[5, :blocksize] = 0.0                                 # an all-zero segment
    tdtype = torch.float32 if dtype == "fp32" else torch.bfloat16
    A_dev = A.cuda().to(tdtype).contiguous()
    A_host = A_dev.float().cpu().numpy()                   # what the kernel sees, exactly, as fp32
    nb = -(-order // blocksize)
    for diagreal in (False, True):
        mid = "_diagreal" if diagreal else ""
        absmax = torch.full((order * nb,), -1.0, device="cuda")
        diag = torch.full((order,), -1.0, device="cuda") if diagreal else None
        out = torch.zeros((order * order * bits + 7) // 8, dtype=torch.uint8, device="cuda")
        quan = getattr(lib, f"cquantize_blockwise{mid}_{bits}bit_{dtype}")
        args = [get_ptr(A_dev), get_ptr(code), ct.c_int32(order), get_ptr(absmax)] + ([get_ptr(diag)] if diagreal else [])
        quan(*args, get_ptr(out), ct.c_int32(blocksize))
        torch.cuda.synchronize()
        want = Q.quantize_c(A_host, code_np, order, blocksize, bits, diagreal)
        assert np.array_equal(out.cpu().numpy(), want[0]), (mid, "codes")
        assert np.array_equal(bits_of(absmax.cpu().numpy()), bits_of(want[1])), (mid, "absmax")
        if diagreal:
            assert np.array_equal(bits_of(diag.cpu().numpy()), bits_of(want[2])), (mid, "diag")
        back = torch.full((order, order), 7.0, dtype=tdtype, device="cuda")
        dequan = getattr(lib, f"cdequantize_blockwise{mid}_{bits}bit_{dtype}")
        args = [get_ptr(out), get_ptr(code), ct.c_int32(order), get_ptr(absmax)] + ([get_ptr(diag)] if diagreal else [])
        dequan(*args, get_ptr(back), ct.c_int32(blocksize))
        torch.cuda.synchronize()
        want_back = Q.dequantize_c(want[0], code_np, order, want[1], blocksize, bits, diag=want[2] if diagreal else None,
                                   to_bf16=dtype == "bf16")
        assert np.array_equal(bits_of(back.float().cpu().numpy()), bits_of(want_back)), (mid, "dequantized")


def test_pipe_switch_and_matrix_pipe_yardstick_through_the_bare_library():
    """The two entry points around the matrix pipes, called as a C program would: the process-wide switch
    (query, set, refuse) and the launch that is nothing but matrix instructions, whose rate must lie between a
    tenth of the published peak and the peak itself on either pipe."""
    lib = ct.cdll.LoadLibrary(str(LIB))
    lib.qtensor_hip_gemm_pipe.restype = ct.c_int
    lib.qtensor_hip_mfma_rate_flop.restype = ct.c_double
    lib.qtensor_hip_mfma_rate_flop.argtypes = [ct.c_int, ct.c_int, ct.c_int, ct.c_void_p, ct.c_void_p]
    lib.qtensor_hip_last_error.restype = ct.c_int
    before = lib.qtensor_hip_gemm_pipe(ct.c_int(-1))
    try:
        assert before in (0, 1)
        assert lib.qtensor_hip_gemm_pipe(ct.c_int(0)) == before and lib.qtensor_hip_gemm_pipe(ct.c_int(-1)) == 0
        assert lib.qtensor_hip_gemm_pipe(ct.c_int(1)) == 0 and lib.qtensor_hip_gemm_pipe(ct.c_int(-1)) == 1
        assert lib.qtensor_hip_gemm_pipe(ct.c_int(7)) == 1 and lib.qtensor_hip_last_error() != 0      # refused, unchanged
        assert lib.qtensor_hip_gemm_pipe(ct.c_int(-1)) == 1 and lib.qtensor_hip_last_error() == 0
    finally:
        lib.qtensor_hip_gemm_pipe(ct.c_int(before))
    sink = torch.zeros(1, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.qtensor_hip_mfma_rate_flop(2, 10, 1, sink.data_ptr(), stream) == 0.0 and lib.qtensor_hip_last_error() != 0
    assert lib.qtensor_hip_mfma_rate_flop(1, 0, 1, sink.data_ptr(), stream) == 0.0 and lib.qtensor_hip_last_error() != 0
    assert lib.qtensor_hip_mfma_rate_flop(1, 10, 1, None, stream) == 0.0 and lib.qtensor_hip_last_error() != 0
    for pipe, rounds, peak in ((1, 4000, 2500e12), (0, 1000, 157.3e12)):
        lib.qtensor_hip_mfma_rate_flop(pipe, rounds, 2, sink.data_ptr(), stream)              # warm-up
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        flop = lib.qtensor_hip_mfma_rate_flop(pipe, rounds, 2, sink.data_ptr(), stream)
        e1.record()
        torch.cuda.synchronize()
        assert lib.qtensor_hip_last_error() == 0 and flop > 0
        rate = flop / (e0.elapsed_time(e1) * 1e-3)
        assert 0.1 * peak <= rate <= 1.02 * peak, (pipe, rate)
    assert float(sink[0]) == 0.0                                                              # the sink is never written
