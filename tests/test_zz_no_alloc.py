"""qtensor_hip_gemm_static -- the entry point for callers that cannot allocate (its split-k partial
products live in a static device array of the library image) -- called through the C ABI and compared
with qtensor_hip_gemm given a caller workspace of the same size: bit for bit, on two calls in a row,
the second with a smaller problem; and with the float64 product (relative Frobenius <= 1e-5)."""
import ctypes as ct

import numpy as np
import pytest
import torch

from oracle import quant_np as Q

pytestmark = pytest.mark.gpu
SCRATCH_FLOATS = 1 << 24


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm())


@pytest.fixture(scope="module")
def api():
    import qtensor.functional as F
    import qtensor.fused as X
    assert torch.cuda.is_available() and F.lib is not None
    lib = ct.CDLL(F.lib._name)                               # plain handle: the C ABI and nothing else
    for name in ("qtensor_hip_gemm", "qtensor_hip_gemm_static"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = [ct.POINTER(X.GemmDesc), ct.c_void_p]
    lib.qtensor_hip_last_error.restype = ct.c_int
    lib.qtensor_hip_last_error_string.restype = ct.c_char_p
    return lib, X


def dense_desc(X, A, B, C, workspace=None):
    d = X.GemmDesc()
    d.M, d.K = A.shape
    d.N = B.shape[1]
    d.batch, d.kind_a, d.kind_b, d.epilogue = 1, X.DENSE, X.DENSE, X.EPI_STORE
    d.args.A, d.args.lda = X.BatchPtr(A.data_ptr(), None, 0), A.stride(0)
    d.args.B, d.args.ldb = X.BatchPtr(B.data_ptr(), None, 0), B.stride(0)
    d.args.C, d.args.ldc = X.BatchPtr(C.data_ptr(), None, 0), C.stride(0)
    if workspace is not None:
        d.args.workspace, d.args.workspace_floats = workspace.data_ptr(), workspace.numel()
    return d


def test_static_scratch_entry_point_equals_the_workspace_entry_point(api, code_maps):
    lib, X = api
    g = torch.Generator().manual_seed(3)
    workspace = torch.empty(SCRATCH_FLOATS, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    # few output tiles, long k: the library cuts k into slices.  The second call is smaller.
    for (m, n, k) in ((768, 1024, 3072), (256, 512, 2048)):
        A, B = torch.randn(m, k, generator=g).cuda(), torch.randn(k, n, generator=g).cuda()
        plain, split, static = (torch.full((m, n), float("nan"), device="cuda") for _ in range(3))
        lib.qtensor_hip_gemm(ct.byref(dense_desc(X, A, B, plain)), stream)
        lib.qtensor_hip_gemm(ct.byref(dense_desc(X, A, B, split, workspace)), stream)
        assert lib.qtensor_hip_last_error() == 0
        lib.qtensor_hip_gemm_static(ct.byref(dense_desc(X, A, B, static)), stream)
        assert lib.qtensor_hip_last_error() == 0, lib.qtensor_hip_last_error_string()
        torch.cuda.synchronize()
        assert torch.equal(static, split)
        assert not torch.equal(split, plain)                 # k really was cut: another summation order
        want = A.double() @ B.double()
        assert rel(static, want) <= 1e-5 and rel(plain, want) <= 1e-5
    # the fused dequantize -> product of the preconditioned gradient (quantized left factor), after the
    # calls above have left their partial products in the static array
    code = code_maps[("linear-2", 4)]
    n, cols = 768, 3072
    L = torch.randn(n, n, generator=g)
    codes, absmax, diag = Q.quantize_c(L.numpy(), code, n, 64, 4, True)
    deq = torch.from_numpy(Q.dequantize_c(codes, code, n, absmax, 64, 4, diag=diag).copy())
    dev = [torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in (codes, absmax, diag)]
    table = torch.from_numpy(code).cuda()
    G = (0.02 * torch.randn(n, cols, generator=g)).cuda()

    def quant_desc(C, ws=None):
        d = X.GemmDesc()
        d.M, d.N, d.K, d.batch = n, cols, n, 1
        d.kind_a, d.kind_b, d.epilogue = X.QUANT4, X.DENSE, X.EPI_STORE
        q = X.QuantRef()
        q.codes, q.absmax, q.diag = (X.BatchPtr(t.data_ptr(), None, 0) for t in dev)
        q.order, q.bs_shift = n, 6
        d.args.Aq = q
        d.args.B, d.args.ldb = X.BatchPtr(G.data_ptr(), None, 0), cols
        d.args.C, d.args.ldc = X.BatchPtr(C.data_ptr(), None, 0), cols
        d.args.code = table.data_ptr()
        if ws is not None:
            d.args.workspace, d.args.workspace_floats = ws.data_ptr(), ws.numel()
        return d

    split, static = torch.empty(n, cols, device="cuda"), torch.empty(n, cols, device="cuda")
    lib.qtensor_hip_gemm(ct.byref(quant_desc(split, workspace)), stream)
    lib.qtensor_hip_gemm_static(ct.byref(quant_desc(static)), stream)
    assert lib.qtensor_hip_last_error() == 0, lib.qtensor_hip_last_error_string()
    torch.cuda.synchronize()
    assert torch.equal(static, split)
    assert rel(static, deq.double() @ G.double().cpu()) <= 1e-5


def test_static_scratch_entry_point_rejects_what_does_not_fit(api, capfd):
    lib, X = api
    stream = torch.cuda.current_stream().cuda_stream
    m = n = 4096                                             # 2 * m * n floats = 2^25 > 2^24
    A, B = torch.zeros(m, 64, device="cuda"), torch.zeros(64, n, device="cuda")
    C = torch.full((m, n), 7.0, device="cuda")
    lib.qtensor_hip_gemm_static(ct.byref(dense_desc(X, A, B, C)), stream)
    assert lib.qtensor_hip_last_error() != 0
    assert b"exceed the static scratch" in lib.qtensor_hip_last_error_string()
    d = dense_desc(X, A[:256], B[:, :256], C)
    d.epilogue = X.EPI_AXPBY_DENSE
    lib.qtensor_hip_gemm_static(ct.byref(d), stream)
    assert lib.qtensor_hip_last_error() != 0
    torch.cuda.synchronize()
    assert bool((C == 7.0).all())                            # nothing was launched
    capfd.readouterr()


def test_static_scratch_entry_point_allocates_nothing_and_refuses_overlapping_calls(api, capfd):
    """The property the entry point exists for: a call (after the first one on the device, which looks the static
    array up) takes no device memory -- the free memory of the device is the same before and after, with torch's
    caching allocator left out of it -- and a call on another stream while the last call's work is still running is
    refused instead of racing on the one shared array."""
    lib, X = api
    g = torch.Generator().manual_seed(4)
    m, n, k = 768, 1024, 3072
    A, B = torch.randn(m, k, generator=g).cuda(), torch.randn(k, n, generator=g).cuda()
    C, C2 = torch.empty(m, n, device="cuda"), torch.empty(m, n, device="cuda")
    main = torch.cuda.current_stream()
    other = torch.cuda.Stream()
    desc, desc2 = dense_desc(X, A, B, C), dense_desc(X, A, B, C2)
    lib.qtensor_hip_gemm_static(ct.byref(desc), main.cuda_stream)                    # warm: symbol looked up, kernels loaded
    assert lib.qtensor_hip_last_error() == 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(3):
        lib.qtensor_hip_gemm_static(ct.byref(desc), main.cuda_stream)
        assert lib.qtensor_hip_last_error() == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    want = C.clone()
    # the same stream again and again: ordered by the stream, never refused
    for _ in range(3):
        lib.qtensor_hip_gemm_static(ct.byref(desc), main.cuda_stream)
        assert lib.qtensor_hip_last_error() == 0
    # another stream while the first one is still busy: refused, nothing launched.  (The first stream is kept busy by
    # work queued ahead of the product: a long elementwise chain.)
    busy = torch.zeros(1 << 26, device="cuda")
    torch.cuda.synchronize()
    for _ in range(40):
        busy.add_(1.0)
    lib.qtensor_hip_gemm_static(ct.byref(desc), main.cuda_stream)
    assert lib.qtensor_hip_last_error() == 0
    with torch.cuda.stream(other):
        C2.fill_(7.0)
    # (no ordering between the two streams: that is the point)
    with torch.cuda.stream(other):
        lib.qtensor_hip_gemm_static(ct.byref(desc2), other.cuda_stream)
        refused = lib.qtensor_hip_last_error() != 0
        message = lib.qtensor_hip_last_error_string()
    torch.cuda.synchronize()
    if refused:
        assert b"still in use" in message
    else:
        # the first stream had already drained when the second call came (a very fast device): then the call is legal
        assert torch.equal(C2, want)
    # once the earlier work is done, the other stream is welcome
    with torch.cuda.stream(other):
        lib.qtensor_hip_gemm_static(ct.byref(desc2), other.cuda_stream)
        assert lib.qtensor_hip_last_error() == 0, lib.qtensor_hip_last_error_string()
    torch.cuda.synchronize()
    assert torch.equal(C2, want) and torch.equal(C, want)
    capfd.readouterr()
