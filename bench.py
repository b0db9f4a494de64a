"""Headline benchmark: 4-bit blockwise quantize + dequantize of a 16384 x 16384 fp32 tensor
(268,435,456 elements, 1 GiB; 99% N(0,1) + 1% outliers of sigma 10; linear-2 table, block 64)
on one MI355X, reported as achieved HBM GB/s over the algorithmic bytes.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-step]

One "step" = one quantize launch + one dequantize launch over the whole tensor, inputs
resident in HBM.  The same JSON line also carries, under "precond_step", the second half of the
metric: ms per full 4-bit Shampoo2 step (eigenbasis variant, coupled-Newton inverse roots) over the
ViT-B/32 weight shapes, with its own roofline entry (the batched product of fp32 matrices that dominates
it: on the bf16 matrix pipe with split operands, fp32-grade results; the fp32 pipe's rate beside it) and the CPU restatement timed on a bounded sample beside it; under "precond_step_naive" the
same for the variant that stores the statistics themselves; under "fused_gemm" the fused
dequantize -> MFMA products deq(L) G deq(R) on both matrix pipes; under "other_formats"
the 8-bit and blocksize-256 variants of the headline tensor.  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (str(ROOT), str(ROOT / "low-bit-shampoo_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0
ORDER = 16384
BLOCK = 64
BITS = 4
BYTES_PER_ELEMENT = 4 + BITS / 8 + 4 / BLOCK      # fp32 in/out + packed code + share of the fp32 maximum
# HBM bytes per launch measured with rocprofv3 FETCH_SIZE / WRITE_SIZE on this workload, scaled by
# the library's plain copy kernel (summary: profiles/quantize_dequantize_16384sq_4bit_bs64_hbm_traffic.txt)
MEASURED_TRAFFIC = {"quantize": 1225675980, "dequantize": 1225393971}
TRAFFIC_SOURCE = ("profiles/quantize_dequantize_16384sq_4bit_bs64_hbm_traffic.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of "
                  "this workload, scaled by the same counters over the library's plain copy kernel; a kept profile, "
                  "not re-measured by this run")


def stress_tensor(torch, order, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(order, order, device="cuda", generator=g)
    mask = torch.rand(order, order, device="cuda", generator=g) < 0.01
    x[mask] *= 10.0
    return x


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(torch, x_slice, code):
    """The reference's CPU code path (per-segment torch loop) on a bounded sample: 1024 rows of
    the same tensor viewed as a 4096 x 4096 matrix (identical segments)."""
    from oracle import quant_loop_torch as QL
    order = 4096
    t0 = time.perf_counter()
    out, absmax = QL.quantize_loop(x_slice, code, order, BLOCK, BITS)
    QL.dequantize_loop(out, code, order, absmax, BLOCK, BITS)
    dt = time.perf_counter() - t0
    nbytes = 2 * BYTES_PER_ELEMENT * order * order
    # informational: the same sample through the scalar C restatement (one core, no Python in the loop)
    strong = None
    try:
        from oracle import quant_np as QN
        xs, cs = x_slice.numpy(), code.numpy()
        t1 = time.perf_counter()
        c_out, c_absmax = QN.quantize_c(xs, cs, order, BLOCK, BITS)
        QN.dequantize_c(c_out, cs, order, c_absmax, BLOCK, BITS)
        dc = time.perf_counter() - t1
        strong = {"value": nbytes / dc / 1e9, "unit": "GB/s", "cores": 1, "seconds": dc,
                  "what": "the same sample through the scalar C restatement (oracle/qoracle.c), one core"}
    except (OSError, ImportError, RuntimeError) as exc:      # the compiled checker is not there: say so, go on
        strong = {"value": None, "what": "scalar C restatement not available: %s" % exc}
    return {
        "strong_cpu_baseline": strong,
        "value": nbytes / dt / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": "rows 0-1023 of the same tensor viewed as 4096x4096 (16,777,216 elements, 262,144 segments), "
                  "quantize+dequantize with the per-segment torch loop of the reference's CPU path",
        "seconds": dt,
        "host_cpus": os.cpu_count(),
        "cpu_model": cpu_model(),
        "torch_threads": torch.get_num_threads(),
    }


def vit_b32_shapes():
    """All 2-D weights of a ViT-Base/32 (12 layers) plus patch embedding and a 100-way head."""
    shapes = []
    for _ in range(12):
        shapes += [(768, 2304), (768, 768), (768, 3072), (3072, 768)]
    return shapes + [(3072, 768), (768, 100)]


STEP_KW = dict(stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1024, prec_bits=4, min_lowbit_size=4096,
               quan_blocksize=64)


def precond_step_gpu(torch, variant="shampoo1"):
    """ms per full 4-bit Shampoo + AdamW step over the ViT-B/32 shapes: statistics every step, inverse 4th
    roots (coupled Newton) every 10th step, preconditioned and norm-grafted update every step.  Ten untimed
    steps bring the preconditioners into use.  variant "shampoo1": the statistics themselves are stored
    quantized; "shampoo2": their eigenvector matrices are (one subspace-iteration step per update).
    Gradients cycle through four independent N(0, 0.02^2) sets, copied into fixed buffers between steps."""
    import importlib
    S = importlib.import_module("optimizers." + variant)

    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()               # what earlier parts of this run still hold: not this workload's
    g = torch.Generator(device="cuda").manual_seed(1)
    params = [torch.nn.Parameter(0.02 * torch.randn(s, device="cuda", generator=g)) for s in vit_b32_shapes()]
    grad_sets = [[0.02 * torch.randn(p.shape, device="cuda", generator=g) for p in params] for _ in range(4)]
    extra = dict(inv_root_mode=1) if variant == "shampoo2" else {}
    opt = S.ShampooAdamW(params, lr=1e-3, weight_decay=0.05, start_prec_step=1, stat_compute_steps=1,
                         prec_compute_steps=10, fused=True, **STEP_KW, **extra)
    for p, gr in zip(params, grad_sets[0]):
        p.grad = gr.clone()
    calls = [0]

    def timed_step():
        torch._foreach_copy_([p.grad for p in params], grad_sets[calls[0] % 4])
        calls[0] += 1
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        opt.step()
        e1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, e0.elapsed_time(e1)

    for _ in range(10):
        timed_step()
    torch.cuda.synchronize()
    resident = torch.cuda.memory_allocated()             # parameters, four gradient sets, optimizer state, kept scratch
    regular, newton = [], []
    peak = {"regular": 0, "roots": 0}
    for i in range(11, 31):
        torch.cuda.reset_peak_memory_stats()
        wall, dev = timed_step()
        (newton if i % 10 == 0 else regular).append((wall, dev))
        kind = "roots" if i % 10 == 0 else "regular"
        peak[kind] = max(peak[kind], torch.cuda.max_memory_allocated())
    mean = lambda xs, k: sum(x[k] for x in xs) / len(xs)          # noqa: E731
    reg, new = mean(regular, 0), mean(newton, 0)
    blocks = sum(((m - 1) // 1024 + 1) * ((n - 1) // 1024 + 1) for m, n in vit_b32_shapes())
    gram_flop = 0                                        # G G^T and G^T G of every block of at most 1024 x 1024
    for m, n in vit_b32_shapes():
        rows = [1024] * ((m - 1) // 1024) + [m - 1024 * ((m - 1) // 1024)]
        cols = [1024] * ((n - 1) // 1024) + [n - 1024 * ((n - 1) // 1024)]
        gram_flop += sum(2 * a * a * b + 2 * a * b * b for a in rows for b in cols)
    more = {}
    if variant == "shampoo2":
        bank = next(iter(opt._fused_cache.values()))["bank"]
        more["matrices_redone_with_library_qr"] = bank.qr_fallbacks
        more["matrices_swept_again_with_replacement"] = bank.qr_repairs
        more["cholesky_qr_rounds_per_stack_and_update"] = round(bank.qr_rounds / (30 * len(bank.per_order)), 2)
        more["subspace_iteration_updates"] = 30 * sum(bank.per_order.values())
    import qtensor.fused as X
    more["gemm_pipe"] = ("products on the %s matrix pipe" %
                         ("bf16 (operands split into three bf16 pieces, six products per fp32 product, fp32 accumulation)"
                          if X.gemm_pipe() == "split" else "fp32"))
    return {
        **more,
        "workload": "ViT-B/32 2-D weights (50 parameters, %d blocks of at most 1024, %d quantized statistics and as many "
                    "preconditioners), fp32 N(0,0.02^2) gradients, 4-bit linear-2 blocksize 64, beta 0.95, statistics "
                    "every step, coupled-Newton inverse 4th roots every 10th step, AdamW update; "
                    "optimizers.%s.ShampooAdamW(fused=True%s)" % (blocks, 2 * blocks, variant,
                                                                   ", inv_root_mode=1" if variant == "shampoo2" else ""),
        "ms_per_step_regular": round(reg, 3),
        "ms_per_step_with_inverse_roots": round(new, 3),
        "ms_per_step_amortized_over_10": round((9 * reg + new) / 10, 3),
        "device_ms_regular": round(mean(regular, 1), 3),
        "device_ms_with_inverse_roots": round(mean(newton, 1), 3),
        "device_memory_gib": {"allocated_between_steps": round((resident - before) / 2 ** 30, 2),
                              "peak_inside_a_step": round((max(peak.values()) - before) / 2 ** 30, 2),
                              "peak_inside_a_regular_step": round((peak["regular"] - before) / 2 ** 30, 2),
                              "peak_inside_a_step_with_inverse_roots": round((peak["roots"] - before) / 2 ** 30, 2),
                              "held_by_earlier_parts_of_the_run_and_left_out": round(before / 2 ** 30, 2),
                              "of_which_parameters_and_the_four_gradient_sets": round(5 * sum(p.numel() for p in params) * 4 / 2 ** 30, 2)},
        "product_gflop_per_regular_step": round(2 * gram_flop / 1e9, 1),
        "product_tflops_regular": round(2 * gram_flop / (mean(regular, 1) * 1e-3) / 1e12, 1),
    }


def per_parameter_layer_gpu(torch, variant="shampoo2", steps=12):
    """The literal drop-in (fused=False: one Preconditioner object per parameter, the reference's own control flow)
    over ONE transformer layer of the ViT-B/32 (qkv, proj, fc1, fc2), same settings as the full step: ms per step.
    Every product of it runs on the library's matrix-core kernels; profile this section to see which kernels it uses."""
    import importlib
    S = importlib.import_module("optimizers." + variant)
    g = torch.Generator(device="cuda").manual_seed(2)
    params = [torch.nn.Parameter(0.02 * torch.randn(s, device="cuda", generator=g)) for s in LAYER_SHAPES]
    grads = [0.02 * torch.randn(p.shape, device="cuda", generator=g) for p in params]
    extra = dict(inv_root_mode=1) if variant == "shampoo2" else {}
    opt = S.ShampooAdamW(params, lr=1e-3, weight_decay=0.05, start_prec_step=1, stat_compute_steps=1,
                         prec_compute_steps=10, fused=False, **STEP_KW, **extra)
    times = []
    for i in range(1, steps + 1):
        for p, gr in zip(params, grads):
            p.grad = gr.clone()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        opt.step()
        torch.cuda.synchronize()
        times.append((i, (time.perf_counter() - t0) * 1e3))
    regular = [t for i, t in times if i % 10 != 0 and i > 2]
    return {"workload": "optimizers.%s.ShampooAdamW(fused=False) over one ViT-B/32 layer (4 parameters, 10 blocks, 20 statistics)" % variant,
            "ms_per_step_regular": round(sum(regular) / len(regular), 3),
            "ms_per_step_with_inverse_roots": round(sum(t for i, t in times if i % 10 == 0) / max(1, sum(1 for i, _ in times if i % 10 == 0)), 3)}


FP32_MATRIX_PEAK_TFLOPS = 157.3
BF16_MATRIX_PEAK_TFLOPS = 2500.0
SPLIT_PRODUCTS = 6            # bf16 products that make one fp32 product on the split pipe
# HBM bytes per launch of the 99 x 1024^3 product (operands 830 MB + result 415 MB algorithmically), kept profile
PRODUCT_TRAFFIC = 1901545267
PRODUCT_TRAFFIC_SOURCE = ("profiles/dense_stack_product_99x1024_kernel_stats_and_mfma_counters.txt: rocprofv3 --pmc FETCH_SIZE / "
                          "WRITE_SIZE of this launch, scaled by the same counters over the library's plain copy kernel; a kept "
                          "profile, not re-measured by this run")


def fused_gemm_gpu(torch, code):
    """deq(Lq) @ G @ deq(Rq) for G 768 x 3072, Lq 768^2 and Rq 3072^2 stored 4-bit / blocksize 64 with exact
    diagonals: the two fused products (three launches), timed with events on the launch stream."""
    import qtensor.fused as X
    g = torch.Generator(device="cuda").manual_seed(3)
    m, n = 768, 3072
    G = 0.02 * torch.randn(m, n, device="cuda", generator=g)

    def inverse_root_like(order):
        q, _ = X.cholesky_qr(torch.randn(1, order, order, device="cuda", generator=g))     # a random orthonormal basis
        q = q[0]
        lam = torch.exp(torch.rand(order, device="cuda", generator=g) * (-6.0 * 2.302585093))   # log-uniform in [1e-6, 1]
        return ((q * lam.pow(-0.25)) @ q.T).contiguous()

    Lq = X.quantize_stack(inverse_root_like(m).unsqueeze(0), X.empty_quantized(1, m, BLOCK, BITS, code, True))
    Rq = X.quantize_stack(inverse_root_like(n).unsqueeze(0), X.empty_quantized(1, n, BLOCK, BITS, code, True))
    half, out = torch.empty(m, n, device="cuda"), torch.empty(m, n, device="cuda")

    def run():
        X.gemm(Lq, G, out=half)
        X.gemm(half, Rq, out=out)

    flop = 2.0 * m * m * n + 2.0 * m * n * n

    def rate():
        # (a hundred untimed runs first: the products are short, and the clock takes tens of milliseconds to settle;
        # then fifty runs back to back between one pair of events, as a step would issue them)
        for _ in range(100):
            run()
        reps = 50
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        return ms, flop / (ms * 1e-3) / 1e12

    before = X.gemm_pipe("f32")
    try:
        ms32, tf32 = rate()
        X.gemm_pipe("split")
        ms, tf = rate()
    finally:
        X.gemm_pipe(before)
    peak = BF16_MATRIX_PEAK_TFLOPS / SPLIT_PRODUCTS
    return {
        "workload": "deq(Lq 768x768) @ G(768x3072) @ deq(Rq 3072x3072), 4-bit linear-2 blocksize 64 factors with exact "
                    "diagonal, expanded inside the two product launches; bf16 MFMA on operands split into three bf16 "
                    "pieces (six products per fp32 product, fp32 accumulation)",
        "ms": round(ms, 4),
        "gflop": round(flop / 1e9, 2),
        "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": round(peak, 1), "unit": "TFLOP/s",
                     "frac": round(tf / peak, 4), "traffic": None,
                     "pipe": "peak = bf16 dense peak %.0f / %d products; achieved counts the algorithmic fp32 flops"
                             % (BF16_MATRIX_PEAK_TFLOPS, SPLIT_PRODUCTS),
                     "achieved_over_fp32_matrix_peak": round(tf / FP32_MATRIX_PEAK_TFLOPS, 4),
                     "fp32_pipe": {"ms": round(ms32, 4), "achieved": round(tf32, 1), "peak": FP32_MATRIX_PEAK_TFLOPS,
                                   "frac": round(tf32 / FP32_MATRIX_PEAK_TFLOPS, 4)}},
    }


def other_formats_gpu(torch, F, x):
    """The same tensor through the other table / blocksize combinations (informational)."""
    n = x.numel()
    out = {}
    for bits, bs in ((4, 256), (8, 64), (8, 256)):
        code = (F.create_linear_map(True, bits, 2) if bits == 4 else F.create_dynamic_map(True, bits, 1)).cuda()
        q = torch.empty(n * bits // 8, dtype=torch.uint8, device="cuda")
        am = torch.empty(n // bs, dtype=torch.float32, device="cuda")
        back = torch.empty_like(x)

        def step():
            F.quantize_blockwise(x, code, ORDER, absmax=am, out=q, blocksize=bs, bits=bits)
            F.dequantize_blockwise(q, code, ORDER, am, out=back, blocksize=bs, bits=bits)

        for _ in range(2):
            step()
        reps = 10
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            step()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        nbytes = 2 * (4 + bits / 8 + 4 / bs) * n
        gbs = nbytes / (ms * 1e-3) / 1e9
        out[f"{bits}bit_bs{bs}"] = {"table": "linear-2" if bits == 4 else "dynamic", "ms_per_step": round(ms, 4),
                                    "GB/s": round(gbs, 1), "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2)}
        del q, am, back
    return out


LAYER_SHAPES = [(768, 2304), (768, 768), (768, 3072), (3072, 768)]


def block_cost(shapes):
    """Sum over the blocks (at most 1024 per side) of m^2 n + m n^2: what the cost of a step is proportional to
    (Gram matrices and applications 2 (m^2 n + m n^2) flop each; the per-statistic work n^3 follows it closely)."""
    total = 0
    for m, n in shapes:
        rows = [1024] * ((m - 1) // 1024) + [m - 1024 * ((m - 1) // 1024)]
        cols = [1024] * ((n - 1) // 1024) + [n - 1024 * ((n - 1) // 1024)]
        total += sum(a * a * b + a * b * b for a in rows for b in cols)
    return total


def precond_step_cpu(torch, code_host, variant):
    """The same regular step (statistics update + preconditioned gradient + norm graft) for ONE transformer
    layer (qkv, proj, fc1, fc2: 10 of the 124 blocks) through the CPU restatement of the reference flow with the
    bit width forced to 4, whose quantizer is the reference's per-segment torch loop."""
    if variant == "shampoo2":
        from oracle.shampoo2_ref import RefPreconditioner2
        make = lambda s: RefPreconditioner2(s, code_host.numpy(), loop=True, inv_root_mode=1, **STEP_KW)   # noqa: E731
    else:
        from oracle.shampoo_ref import RefPreconditioner
        make = lambda s: RefPreconditioner(s, code_host.numpy(), loop=True, **STEP_KW)                     # noqa: E731
    g = torch.Generator().manual_seed(1)
    grads = [0.02 * torch.randn(s, generator=g) for s in LAYER_SHAPES]
    pres = [make(s) for s in LAYER_SHAPES]
    t0 = time.perf_counter()
    for pre, gr in zip(pres, grads):
        pre.add_statistics(gr)
        out = pre.preconditioned_grad(gr)
        out.mul_(gr.norm() / (out.norm() + 1e-12))
    regular = time.perf_counter() - t0
    factor = block_cost(vit_b32_shapes()) / block_cost(LAYER_SHAPES)
    return {
        "value": round(regular * 1e3 * factor, 1),
        "unit": "ms per regular step, EXTRAPOLATED from the sample by the ratio %.2f of sum(m^2 n + m n^2) over the blocks" % factor,
        "kind": "port",
        "cores": torch.get_num_threads(),
        "sample": "one transformer layer (4 of 50 parameters, 10 of 124 blocks, 20 of 248 statistics): statistics "
                  "update + preconditioned gradient + norm graft through oracle/%s; quantizer = per-segment torch "
                  "loop (1 core), products%s = torch on %d threads"
                  % ("shampoo2_ref.py" if variant == "shampoo2" else "shampoo_ref.py",
                     " and QR" if variant == "shampoo2" else "", torch.get_num_threads()),
        "seconds_for_sample": round(regular, 3),
    }


def dominant_product_gpu(torch):
    """The kernel most of a step's time goes to -- gemm_kernel<128,128,dense,dense,store>, the batched plain product
    of fp32 matrices (L Q, the Newton products, the projections of the Gram-Schmidt sweep) -- on the step's biggest
    stack (99 statistics of order 1024), timed per launch with events on the launch stream, on both matrix pipes.
    The default pipe splits every fp32 operand into three bf16 pieces and takes six bf16 MFMA products per fp32
    product (fp32 accumulation, fp32-grade results): its roofline is the bf16 matrix peak over six."""
    import qtensor.fused as X
    g = torch.Generator(device="cuda").manual_seed(5)
    batch, n = 99, 1024
    A = torch.randn(batch, n, n, device="cuda", generator=g)
    B = torch.randn(batch, n, n, device="cuda", generator=g)
    C = torch.empty(batch, n, n, device="cuda")
    flop = 2.0 * batch * n ** 3
    reps = 10

    def rate():
        for _ in range(20):                      # the clocks settle over the first dozen launches
            X.gemm(A, B, out=C)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        ev[0].record()
        for i in range(reps):
            X.gemm(A, B, out=C)
            ev[i + 1].record()
        torch.cuda.synchronize()
        ms = sum(ev[i].elapsed_time(ev[i + 1]) for i in range(reps)) / reps
        return ms, flop / (ms * 1e-3) / 1e12

    def pipe_alone(pipe):
        """TFLOP/s of a launch that is nothing but matrix instructions on register operands of random bits."""
        import ctypes as ct
        import qtensor.functional as F
        F.lib.qtensor_hip_mfma_rate_flop.restype = ct.c_double
        F.lib.qtensor_hip_mfma_rate_flop.argtypes = [ct.c_int, ct.c_int, ct.c_int, ct.c_void_p, ct.c_void_p]
        sink = torch.zeros(1, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream
        rounds = 20000 if pipe == 1 else 5000
        F.lib.qtensor_hip_mfma_rate_flop(pipe, rounds, 3, sink.data_ptr(), stream)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        done = F.lib.qtensor_hip_mfma_rate_flop(pipe, rounds, 3, sink.data_ptr(), stream)
        e1.record()
        torch.cuda.synchronize()
        return done / (e0.elapsed_time(e1) * 1e-3) / 1e12

    before = X.gemm_pipe("f32")
    try:
        ms32, tf32 = rate()
        X.gemm_pipe("split")
        ms, tf = rate()
    finally:
        X.gemm_pipe(before)
    peak = BF16_MATRIX_PEAK_TFLOPS / SPLIT_PRODUCTS
    return {"bound": "mfma", "kernel": "gemm_kernel<128,128,dense,dense,store,split> on 99 x (1024 x 1024 x 1024)",
            "achieved": round(tf, 1), "peak": round(peak, 1), "unit": "TFLOP/s", "frac": round(tf / peak, 4),
            "traffic": PRODUCT_TRAFFIC, "traffic_source": PRODUCT_TRAFFIC_SOURCE,
            "avg_launch_ms": round(ms, 4), "algorithmic_flop_per_launch": flop,
            "pipe": "v_mfma_f32_32x32x16_bf16 on operands split into three bf16 pieces: %d bf16 products per fp32 product, "
                    "so peak = bf16 dense peak %.0f / %d; achieved counts the algorithmic fp32 flops (2 m n k)"
                    % (SPLIT_PRODUCTS, BF16_MATRIX_PEAK_TFLOPS, SPLIT_PRODUCTS),
            "bf16_mfma_tflops": round(tf * SPLIT_PRODUCTS, 1),
            "matrix_instructions_alone": {
                "what": "one launch of nothing but matrix instructions on register operands of random bits, three "
                        "workgroups per compute unit: the rate each pipe sustains at the clock it holds under that load",
                "bf16_tflops": round(pipe_alone(1), 1), "fp32_tflops": round(pipe_alone(0), 1)},
            "fp32_pipe": {"kernel": "gemm_kernel<128,128,dense,dense,store> (v_mfma_f32_32x32x2_f32)", "achieved": round(tf32, 1),
                          "peak": FP32_MATRIX_PEAK_TFLOPS, "frac": round(tf32 / FP32_MATRIX_PEAK_TFLOPS, 4),
                          "avg_launch_ms": round(ms32, 4)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--section", choices=["all", "quant", "gemm", "step", "step2", "product", "layer"], default="all",
                    help="run only one part (for profiling one kernel family); the JSON line then lacks the others")
    ap.add_argument("--bank-streams", type=int, default=None,
                    help="side streams of the batched preconditioner engine (0 serialises its launches, which "
                         "keeps per-kernel durations in a profile free of overlap)")
    ap.add_argument("--gemm-pipe", choices=["f32", "split"], default=None,
                    help="matrix pipe of the products of dense operands (default: the library's, the split bf16 pipe)")
    ap.add_argument("--no-step", action="store_true", help="skip the fused-product, other-format and Shampoo-step measurements")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).")

    import torch
    import qtensor.functional as F

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU.")
    if F.lib is None:
        sys.exit("libqtensor_hip.so is missing; run `python -c 'import __graft_entry__ as g; g.build()'`.")

    code_host = F.create_linear_map(True, BITS, 2)
    code = code_host.cuda()
    if args.gemm_pipe is not None:
        import qtensor.fused as X
        X.gemm_pipe(args.gemm_pipe)
    if args.bank_streams is not None:
        from optimizers.engine import ShampooBank
        from optimizers.engine2 import ShampooBank2
        ShampooBank.DEFAULT_STREAMS = ShampooBank2.DEFAULT_STREAMS = args.bank_streams
        if args.bank_streams == 0:           # profiling: nothing may overlap, the side thread of shampoo2 neither
            from optimizers import shampoo2
            shampoo2.ShampooAdamW.overlap_precondition = False
    if args.section in ("gemm", "step", "step2", "product", "layer"):
        if args.section == "layer":
            part = {"per_parameter_layer": per_parameter_layer_gpu(torch)}
        elif args.section == "gemm":
            part = {"fused_gemm": fused_gemm_gpu(torch, code)}
        elif args.section == "step":
            part = {"precond_step_naive": precond_step_gpu(torch)}
        elif args.section == "product":
            part = {"roofline": dominant_product_gpu(torch)}
        else:
            part = {"precond_step": precond_step_gpu(torch, "shampoo2")}
        print(json.dumps({"section": args.section, "n_gpus": 1, **part}))
        return
    if args.section == "quant":
        args.no_step = args.no_cpu_baseline = True
    x = stress_tensor(torch, ORDER)
    n = ORDER * ORDER
    out = torch.empty(n * BITS // 8, dtype=torch.uint8, device="cuda")
    absmax = torch.empty(n // BLOCK, dtype=torch.float32, device="cuda")
    back = torch.empty(ORDER, ORDER, dtype=torch.float32, device="cuda")

    # One copy of the same tensor through the library's plain copy kernel, outside the timed
    # region: profiler byte counters are scaled against its exactly known traffic (1 GiB each way).
    import ctypes as ct
    F.lib.qtensor_hip_copy_f32.restype = None
    F.lib.qtensor_hip_copy_f32.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_ulonglong, ct.c_void_p]
    F.lib.qtensor_hip_copy_f32(x.data_ptr(), back.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    def step():
        F.quantize_blockwise(x, code, ORDER, absmax=absmax, out=out, blocksize=BLOCK, bits=BITS)
        F.dequantize_blockwise(out, code, ORDER, absmax, out=back, blocksize=BLOCK, bits=BITS)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3

    # per-kernel durations with events on the launch stream (torch's current stream)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    for e0, e1, e2 in ev:
        e0.record()
        F.quantize_blockwise(x, code, ORDER, absmax=absmax, out=out, blocksize=BLOCK, bits=BITS)
        e1.record()
        F.dequantize_blockwise(out, code, ORDER, absmax, out=back, blocksize=BLOCK, bits=BITS)
        e2.record()
    torch.cuda.synchronize()
    q_ms = sum(e0.elapsed_time(e1) for e0, e1, _ in ev) / args.steps
    d_ms = sum(e1.elapsed_time(e2) for _, e1, e2 in ev) / args.steps

    algo = BYTES_PER_ELEMENT * n                     # per launch, same for quantize and dequantize
    value = 2 * algo / (ms_per_step * 1e-3) / 1e9
    q_gbs = algo / (q_ms * 1e-3) / 1e9
    d_gbs = algo / (d_ms * 1e-3) / 1e9
    result = {
        "metric": "quant+dequant HBM GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "16384x16384 fp32 (99% N(0,1), 1% sigma-10 outliers), 4-bit linear-2 table, "
                        "blocksize 64: blockwise quantize then dequantize of the whole tensor",
            "elements": n,
            "algorithmic_bytes_per_step": int(2 * algo),
        },
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "roofline": {
            "bound": "hbm",
            "kernel": "quantize_flat_kernel<float,4,64,false,true,true>",
            "achieved": round(q_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(q_gbs / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC["quantize"],
            "traffic_source": TRAFFIC_SOURCE,
            "avg_launch_ms": round(q_ms, 4),
            "algorithmic_bytes_per_launch": int(algo),
        },
        "dequantize": {
            "kernel": "dequantize_flat_kernel<float,4,false,true>",
            "traffic": MEASURED_TRAFFIC["dequantize"],
            "achieved": round(d_gbs, 1),
            "frac": round(d_gbs / HBM_PEAK_GBS, 4),
            "avg_launch_ms": round(d_ms, 4),
        },
    }
    x_slice = None if args.no_cpu_baseline else x.view(-1)[: 4096 * 4096].cpu()
    del out, absmax, back
    if not args.no_step:
        result["other_formats"] = other_formats_gpu(torch, F, x)
    del x
    torch.cuda.empty_cache()
    if not args.no_step:
        result["fused_gemm"] = fused_gemm_gpu(torch, code)
        # the step the headline configuration names: eigenbasis variant with coupled-Newton inverse roots
        result["precond_step"] = precond_step_gpu(torch, "shampoo2")
        result["precond_step"]["roofline"] = dominant_product_gpu(torch)
        result["precond_step_naive"] = precond_step_gpu(torch, "shampoo1")
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, x_slice, code_host)
        if not args.no_step:
            for key, variant in (("precond_step", "shampoo2"), ("precond_step_naive", "shampoo1")):
                cpu = precond_step_cpu(torch, code_host, variant)
                result[key]["cpu_baseline"] = cpu
                result[key]["speedup_vs_extrapolated_cpu_regular_step"] = round(
                    cpu["value"] / result[key]["ms_per_step_regular"], 1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
