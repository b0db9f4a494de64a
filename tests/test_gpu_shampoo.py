"""GPU parity of the low-bit preconditioner step: the per-parameter Preconditioner (reference
layout), the batched ShampooBank and the fused optimizer, against the CPU restatement with the
quantizer oracle (oracle/shampoo_ref.py) on identical gradients and start vectors.

Tolerances.  One fused statistics update differs from the CPU flow only by fp32 summation order
inside the products (~1e-7 relative), so after quantization almost every code agrees; a code can
flip where a quotient sits within that distance of a decision threshold.  Bounds used: at most
0.1 % of codes differ after three updates; dequantized statistics within 1e-3, preconditioned
gradients within 2e-3 relative Frobenius norm.  Bank against per-parameter path (same kernels,
same start vectors): bit-identical statistics, inverse roots equal to rounding."""
import numpy as np
import pytest
import torch

from oracle.shampoo_ref import RefPreconditioner

pytestmark = pytest.mark.gpu
SHAPES = [(128, 192), (256, 64), (64,), (192, 1, 128)]
KW = dict(stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=128, prec_bits=4, min_lowbit_size=4096, quan_blocksize=64)


def rel(a, b):
    a, b = torch.as_tensor(a).double().cpu(), torch.as_tensor(b).double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


@pytest.fixture(scope="module")
def setup(code_maps):
    import qtensor.functional as F
    from optimizers import shampoo1 as S1
    from optimizers.engine import ShampooBank
    assert torch.cuda.is_available() and F.lib is not None
    g = torch.Generator().manual_seed(11)
    grads = [[0.02 * torch.randn(s, generator=g) for s in SHAPES] for _ in range(3)]
    return S1, ShampooBank, grads, code_maps[("linear-2", 4)]


def start_vectors(step, orders):
    g = torch.Generator().manual_seed(500 + step)
    return [torch.rand(o, generator=g) * 2 - 1 for o in orders]


def test_per_parameter_low_bit_path_follows_the_oracle(setup):
    S1, _, grads, code = setup
    for k, shape in enumerate(SHAPES):
        ref = RefPreconditioner(shape, code, **KW)
        qmap = {"linear-2": torch.from_numpy(code)}
        pre = S1.Preconditioner(torch.zeros(shape, device="cuda"), qmap, **KW)
        assert len(pre.statistics) == len(ref.stats)
        orders = [s.order for s in ref.stats]
        for st in range(3):
            grad = grads[st][k]
            ref.add_statistics(grad)
            pre.add_statistics(grad.cuda())
            v0 = start_vectors(st, orders)
            ref.compute_preconditioners(v0)
            pre.compute_preconditioners([v.cuda() for v in v0])
            out = pre.preconditioned_grad(grad.cuda())
            want = ref.preconditioned_grad(grad)
            assert out.shape == grad.shape
            assert rel(out, want) <= 2e-3, (shape, st)
        for h, slot in zip(pre.statistics, ref.stats):
            assert h.bits == 4 and slot.low
            codes, absmax, diag = slot.codes()
            got = h.var.cpu().numpy()
            differing = np.count_nonzero((got >> 4) != (codes >> 4)) + np.count_nonzero((got & 15) != (codes & 15))
            assert differing <= 1e-3 * 2 * got.size
            assert rel(h.absmax, absmax) <= 1e-5 and rel(h.diag, diag) <= 1e-5
            assert rel(h.dequantize(), slot.get()) <= 1e-3
        for h, slot in zip(pre.preconditioners, ref.precs):
            assert rel(h.dequantize(), slot.get()) <= 2e-3


@pytest.mark.parametrize("bits", [4, 8])
def test_bank_equals_per_parameter_path(setup, code_maps, bits):
    S1, ShampooBank, grads, code = setup
    code = code_maps[("linear-2", bits)]
    KW = dict(globals()["KW"], prec_bits=bits)
    mats = [s for s in SHAPES if len([d for d in s if d != 1]) > 1]
    params = [torch.zeros(s, device="cuda") for s in mats]
    kw = {k: v for k, v in KW.items() if k in ("prec_maxorder", "prec_bits", "min_lowbit_size", "quan_blocksize")}
    assert all(ShampooBank.accepts(p, **kw) for p in params)
    assert not ShampooBank.accepts(torch.zeros(64, device="cuda"), **kw)             # a vector has no statistics
    assert ShampooBank.accepts(torch.zeros(128, 100, device="cuda"), **kw)           # 100 is not a multiple of 64: general layout
    assert ShampooBank.accepts(torch.zeros(96, 40, device="cuda"), **kw)             # 40 x 40 is below min_lowbit_size: kept in fp32
    assert not ShampooBank.accepts(torch.zeros(128, 128), **kw)                      # CPU
    assert not ShampooBank.accepts(torch.zeros(128, 128, device="cuda", dtype=torch.bfloat16), **kw)
    qmap = {"linear-2": torch.from_numpy(code)}
    bank = ShampooBank(params, qmap, "linear-2", **KW)
    pres = [S1.Preconditioner(p, qmap, **KW) for p in params]
    table = bank.block_table()
    assert len(table) == sum(len(p.statistics) for p in pres)
    idx = [SHAPES.index(s) for s in mats]
    for st in range(3):
        gl = [grads[st][i].cuda() for i in idx]
        bank.add_statistics(gl)
        v0_bank = {o: torch.empty(q.batch, o) for o, q in bank.stats.items()}
        v0_pre = []
        for pi, pre in enumerate(pres):
            pre.add_statistics(gl[pi])
            orders = [h.var_order for h in pre.statistics]
            vs = start_vectors(st * 10 + pi, orders)
            v0_pre.append(vs)
            for (tpi, j, side, order, row) in table:
                if tpi == pi:
                    v0_bank[order][row] = vs[2 * j + side]
        bank.compute_preconditioners({o: v.cuda() for o, v in v0_bank.items()})
        outs = bank.preconditioned_grads(gl)
        for pi, pre in enumerate(pres):
            pre.compute_preconditioners([v.cuda() for v in v0_pre[pi]])
            want = pre.preconditioned_grad(gl[pi])
            assert outs[pi].shape == want.shape
            assert rel(outs[pi], want) <= (1e-4 if bits == 4 else 5e-4)      # more, smaller code flips on the finer grid
    for (pi, j, side, order, row) in table:
        h = pres[pi].statistics[2 * j + side]              # statistics: same kernels, bit-identical
        assert torch.equal(bank.stats[order].codes[row], h.var)
        assert torch.equal(bank.stats[order].absmax[row], h.absmax)
        assert torch.equal(bank.stats[order].diag[row], h.diag)
        # inverse roots: torch's batched reductions (norms, matrix-vector products) round differently
        # for a stack of one and a stack of many, so agreement is to rounding, not to the bit
        h = pres[pi].preconditioners[2 * j + side]
        got, want = bank.precs[order].codes[row], h.var
        differing = int(((got >> 4) != (want >> 4)).sum() + ((got & 15) != (want & 15)).sum()) if bits == 4 else int((got != want).sum())
        assert differing <= (1e-3 * 2 if bits == 4 else 2e-2) * got.numel()      # 8-bit steps are 16 times finer
        assert rel(bank.precs[order].absmax[row], h.absmax) <= 1e-5
        assert rel(bank.precs[order].diag[row], h.diag) <= 1e-5
    sd = bank.state_dict()
    bank2 = ShampooBank(params, qmap, "linear-2", **KW)
    bank2.load_state_dict(sd)
    first = outs[0].clone()
    assert bank2.is_active() and torch.equal(bank2.preconditioned_grads(gl)[0], first)


@pytest.mark.parametrize("which", ["adamw", "sgd"])
def test_fused_optimizer_matches_per_parameter_optimizer(setup, which, monkeypatch):
    S1, _, grads, _ = setup
    import optimizers.matrix_functions as MF
    real_rand = torch.rand
    # identical, deterministic power-iteration start vectors on both paths
    monkeypatch.setattr(MF.torch, "rand", lambda *size, **kw: torch.full(size, 0.75, **kw))
    shapes = SHAPES + [(128, 100), (96, 40)]           # orders the blocksize does not divide / too small to quantize
    g = torch.Generator().manual_seed(5)
    init = [real_rand(s, generator=g) for s in shapes]
    gs = [[0.02 * torch.randn(s, generator=g) for s in shapes] for _ in range(4)]
    finals = []
    for fused in (False, True):
        params = [torch.nn.Parameter(t.clone().cuda()) for t in init]
        common = dict(start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2, fused=fused, **KW)
        opt = (S1.ShampooAdamW(params, lr=1e-2, weight_decay=0.05, **common) if which == "adamw"
               else S1.ShampooSGD(params, lr=1e-2, momentum=0.9, weight_decay=1e-3, nesterov=True, **common))
        for st in range(4):
            for p, gr in zip(params, gs[st]):
                p.grad = gr.clone().cuda()
            opt.step()
        finals.append([p.detach().cpu() for p in params])
    # four steps of size lr = 1e-2 on O(1) parameters; the two paths agree to a small fraction of one
    # update (Adam's normalisation magnifies the rounding-level differences of the inverse roots)
    for a, b in zip(*finals):
        assert rel(a, b) <= 2e-4


@pytest.mark.parametrize("which", ["adamw", "sgd", "sgd-nesterov"])
def test_fused_update_kernels_match_the_torch_update_rules(which):
    """Grafting + AdamW / SGD update of all tensors in two launches against the reference's torch
    calls (shampoo1.py:310-331, 405-427) on ragged, unaligned and multi-chunk tensors."""
    import math
    from optimizers.tail import TailPlan
    g = torch.Generator().manual_seed(11)
    sizes = [5, 16384, 16385, 100003, 3 * 16384 + 2, 1]
    graft = [True, True, False, True, True, True]
    pool = torch.randn(sum(sizes) + 64, generator=g).cuda()

    def carve(unaligned):
        out, at = [], 1 if unaligned else 0
        for n in sizes:
            out.append(pool[at:at + n].clone() if not unaligned else torch.randn(n + 1, generator=g).cuda()[1:])
            at += n
        return out

    for unaligned in (False, True):
        params, dirs, grads = carve(unaligned), carve(unaligned), carve(unaligned)
        m = [0.1 * torch.randn(n, generator=g).cuda() for n in sizes]
        v = [0.01 * torch.rand(n, generator=g).cuda() for n in sizes]
        want_p, want_m, want_v = [t.clone() for t in params], [t.clone() for t in m], [t.clone() for t in v]
        lr, wd, step = 1e-2, 0.05, 3
        plan = TailPlan()
        for p, d, gr, a, b, f in zip(want_p, dirs, grads, want_m, want_v, graft):
            d = d.clone()
            if f:
                d.mul_(gr.norm() / (d.norm() + 1e-12))
            if which == "adamw":
                beta1, beta2, eps = 0.9, 0.999, 1e-8
                p.mul_(1 - lr * wd)
                a.mul_(beta1).add_(d, alpha=1 - beta1)
                b.mul_(beta2).addcmul_(d, d, value=1 - beta2)
                denom = (b.sqrt() / math.sqrt(1 - beta2 ** step)).add_(eps)
                p.addcdiv_(a, denom, value=-lr / (1 - beta1 ** step))
            else:
                d.add_(p, alpha=wd)
                buf = a.mul_(0.9).add_(d)
                p.add_(d.add(buf, alpha=0.9) if which == "sgd-nesterov" else buf, alpha=-lr)
        before = [d.clone() for d in dirs]
        if which == "adamw":
            plan.adamw(params, dirs, grads, m, v, graft, lr, (0.9, 0.999), 1e-8, wd, step)
        else:
            plan.sgd(params, dirs, grads, m, graft, lr, 0.9, wd, which == "sgd-nesterov")
        for got, want in zip(params + m + (v if which == "adamw" else []), want_p + want_m + (want_v if which == "adamw" else [])):
            assert rel(got, want) <= 2e-6
        assert all(torch.equal(a, b) for a, b in zip(dirs, before))      # directions are read only
        # the plan is reused while no buffer moves, and rebuilt when one does
        table = plan.table
        (plan.adamw(params, dirs, grads, m, v, graft, lr, (0.9, 0.999), 1e-8, wd, step + 1) if which == "adamw"
         else plan.sgd(params, dirs, grads, m, graft, lr, 0.9, wd, False))
        assert plan.table is table
    with pytest.raises(ValueError):
        TailPlan().sgd([torch.zeros(4, device="cuda")], [torch.zeros(4)], [torch.zeros(4, device="cuda")],
                       [torch.zeros(4, device="cuda")], [False], 0.1, 0.9, 0.0, False)


@pytest.mark.parametrize("which", ["adamw", "sgd"])
def test_fused_optimizer_checkpoint_round_trip(setup, which, monkeypatch):
    """state_dict() of the fused optimizers carries the bank's quantized state as plain tensors: a run
    resumed from a checkpoint (written and read with weights_only=True for the bank part) continues
    exactly like the uninterrupted one."""
    import io
    S1 = setup[0]
    import optimizers.matrix_functions as MF
    real_rand = torch.rand
    monkeypatch.setattr(MF.torch, "rand", lambda *size, **kw: torch.full(size, 0.75, **kw))
    g = torch.Generator().manual_seed(6)
    init = [real_rand(s, generator=g) for s in SHAPES]
    gs = [[0.02 * torch.randn(s, generator=g) for s in SHAPES] for _ in range(5)]

    def make(params):
        common = dict(start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2, fused=True, **KW)
        return (S1.ShampooAdamW(params, lr=1e-2, weight_decay=0.05, **common) if which == "adamw"
                else S1.ShampooSGD(params, lr=1e-2, momentum=0.9, **common))

    def run(opt, params, steps):
        for st in steps:
            for p, gr in zip(params, gs[st]):
                p.grad = gr.clone().cuda()
            opt.step()

    straight = [torch.nn.Parameter(t.clone().cuda()) for t in init]
    run(make(straight), straight, range(5))

    first = [torch.nn.Parameter(t.clone().cuda()) for t in init]
    opt = make(first)
    run(opt, first, range(3))
    sd = opt.state_dict()
    bank = sd["shampoo_bank"]
    assert len(bank) == 1 and bank[0]["block_table"].shape[1] == 5
    assert all(isinstance(v, torch.Tensor) for v in bank[0].values())
    assert all(opt.state[p]["step"] == 3 for p in first)
    assert not any("preconditioner" in opt.state[p] for p in first if p.dim() > 1)      # every matrix lives in the bank
    buf = io.BytesIO()
    torch.save(sd, buf)                                   # the WHOLE state: nothing in it is a pickled object
    buf.seek(0)
    sd = torch.load(buf, weights_only=True, map_location="cpu")
    resumed = [torch.nn.Parameter(p.detach().clone()) for p in first]
    opt2 = make(resumed)
    opt2.load_state_dict(sd)
    run(opt2, resumed, range(3, 5))
    for a, b in zip(straight, resumed):
        assert torch.equal(a.detach(), b.detach())
    # a checkpoint for other shapes is refused
    other = [torch.nn.Parameter(torch.zeros(128, 64, device="cuda"))]
    opt3 = make(other)
    bad = opt3.state_dict()
    bad["shampoo_bank"] = sd["shampoo_bank"]
    opt3.load_state_dict(bad)
    other[0].grad = torch.ones(128, 64, device="cuda")
    with pytest.raises(ValueError):
        opt3.step()


@pytest.mark.parametrize("which", ["adamw", "sgd"])
def test_fused_step_skips_and_counts_per_parameter_like_the_reference(setup, which, monkeypatch):
    """A parameter without a gradient is skipped and every parameter counts its own steps (reference:
    optimizers/shampoo1.py:371-377, 394-396): the fused step with gradients missing on some steps against the
    per-parameter optimizer on the same gradients."""
    S1 = setup[0]
    import optimizers.matrix_functions as MF
    real_rand = torch.rand
    monkeypatch.setattr(MF.torch, "rand", lambda *size, **kw: torch.full(size, 0.75, **kw))
    shapes = SHAPES + [(128, 100)]
    g = torch.Generator().manual_seed(15)
    init = [real_rand(s, generator=g) for s in shapes]
    gs = [[0.02 * torch.randn(s, generator=g) for s in shapes] for _ in range(7)]
    # which parameters have a gradient at which step: the second one joins late, the first one pauses twice,
    # the vector pauses once, the last one is there every other step
    present = [[st not in (2, 3), st >= 2, st != 4, True, st % 2 == 0] for st in range(7)]
    finals, counts = [], []
    for fused in (False, True):
        params = [torch.nn.Parameter(t.clone().cuda()) for t in init]
        common = dict(start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2, fused=fused, **KW)
        opt = (S1.ShampooAdamW(params, lr=1e-2, weight_decay=0.05, **common) if which == "adamw"
               else S1.ShampooSGD(params, lr=1e-2, momentum=0.9, weight_decay=1e-3, **common))
        for st in range(7):
            for p, gr, there in zip(params, gs[st], present[st]):
                p.grad = gr.clone().cuda() if there else None
            opt.step()
        finals.append([p.detach().cpu() for p in params])
        counts.append([opt.state[p]["step"] for p in params])
    assert counts[0] == counts[1] == [sum(row[k] for row in present) for k in range(len(shapes))]
    for a, b in zip(*finals):
        assert rel(a, b) <= 2e-4


def test_fused_step_error_paths(setup):
    """What the fused optimizer refuses."""
    S1 = setup[0]
    g = torch.Generator().manual_seed(8)
    params = [torch.nn.Parameter(torch.rand(s, generator=g).cuda()) for s in SHAPES]
    opt = S1.ShampooAdamW(params, lr=1e-2, start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2, fused=True, **KW)
    for p in params:
        p.grad = 0.02 * torch.randn(p.shape, generator=g).cuda()
    opt.step()
    assert all(opt.state[p]["step"] == 1 for p in params)
    # a checkpoint of the fused optimizer does not load into the per-parameter one
    sd = opt.state_dict()
    plain = S1.ShampooAdamW([torch.nn.Parameter(p.detach().clone()) for p in params], lr=1e-2, start_prec_step=2,
                            stat_compute_steps=1, prec_compute_steps=2, fused=False, **KW)
    with pytest.raises(ValueError, match="fused=True"):
        plain.load_state_dict(sd)
    # more blocks of one order than one launch takes
    from optimizers.engine import ShampooBank
    import qtensor.functional as F
    many = [torch.nn.Parameter(torch.zeros(64 * 65536, 64, device="meta"))]
    with pytest.raises((ValueError, NotImplementedError, RuntimeError)):
        ShampooBank(many, {"code": F.create_linear_map(True, 4, 2)}, "code", prec_maxorder=64, prec_bits=4, min_lowbit_size=4096,
                    quan_blocksize=64)


def test_per_parameter_optimizer_checkpoint_is_flat(setup, monkeypatch):
    """fused=False: state_dict() moves the Preconditioner objects out of the per-parameter state into their flat form
    (tensors, numbers, lists), so the whole checkpoint loads with weights_only=True, and a resumed run continues
    bit for bit."""
    import io
    S1 = setup[0]
    import optimizers.matrix_functions as MF
    real_rand = torch.rand
    monkeypatch.setattr(MF.torch, "rand", lambda *size, **kw: torch.full(size, 0.75, **kw))
    shapes = SHAPES + [(128, 100), (96, 40)]
    g = torch.Generator().manual_seed(16)
    init = [real_rand(s, generator=g) for s in shapes]
    gs = [[0.02 * torch.randn(s, generator=g) for s in shapes] for _ in range(5)]

    def make(params):
        return S1.ShampooAdamW(params, lr=1e-2, weight_decay=0.05, start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2,
                               fused=False, **KW)

    def run(opt, params, steps):
        for st in steps:
            for p, gr in zip(params, gs[st]):
                p.grad = gr.clone().cuda()
            opt.step()

    straight = [torch.nn.Parameter(t.clone().cuda()) for t in init]
    run(make(straight), straight, range(5))
    first = [torch.nn.Parameter(t.clone().cuda()) for t in init]
    opt = make(first)
    run(opt, first, range(3))
    sd = opt.state_dict()
    assert len(sd["shampoo_preconditioners"]) == len(shapes)
    assert not any("preconditioner" in one for one in sd["state"].values())
    assert all("preconditioner" in opt.state[p] for p in first)                      # the live state is untouched
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    sd = torch.load(buf, weights_only=True, map_location="cpu")
    resumed = [torch.nn.Parameter(p.detach().clone()) for p in first]
    opt2 = make(resumed)
    opt2.load_state_dict(sd)
    run(opt2, resumed, range(3, 5))
    for a, b in zip(straight, resumed):
        assert torch.equal(a.detach(), b.detach())


def test_fused_step_with_parameters_the_bank_does_not_take(setup, monkeypatch):
    """A bf16 matrix and a vector stay outside the bank (per-parameter preconditioner, torch's update rules with
    per-parameter bias corrections) next to banked fp32 matrices; gradients are missing on some steps.  Against the
    per-parameter optimizer; the checkpoint stays flat."""
    import io
    S1 = setup[0]
    import optimizers.matrix_functions as MF
    g = torch.Generator().manual_seed(23)
    shapes = [(128, 192), (128, 64), (64,), (256, 64)]
    dtypes = [torch.float32, torch.bfloat16, torch.float32, torch.float32]
    init = [torch.rand(s, generator=g).to(d) for s, d in zip(shapes, dtypes)]
    gs = [[(0.02 * torch.randn(s, generator=g)).to(d) for s, d in zip(shapes, dtypes)] for _ in range(5)]
    present = [[True, st != 1, st != 3, st >= 1] for st in range(5)]
    monkeypatch.setattr(MF.torch, "rand", lambda *size, **kw: torch.full(size, 0.75, **kw))
    finals = []
    for fused in (False, True):
        params = [torch.nn.Parameter(t.clone().cuda()) for t in init]
        opt = S1.ShampooAdamW(params, lr=1e-2, weight_decay=0.05, start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2,
                              fused=fused, **KW)
        for st in range(5):
            for p, gr, there in zip(params, gs[st], present[st]):
                p.grad = gr.clone().cuda() if there else None
            opt.step()
        finals.append([p.detach().float().cpu() for p in params])
        if fused:
            assert "preconditioner" in opt.state[params[1]] and "preconditioner" in opt.state[params[2]]
            assert "preconditioner" not in opt.state[params[0]] and "preconditioner" not in opt.state[params[3]]
            sd = opt.state_dict()
            assert sorted(sd["shampoo_preconditioners"]) == [1, 2]
            buf = io.BytesIO()
            torch.save(sd, buf)
            buf.seek(0)
            torch.load(buf, weights_only=True, map_location="cpu")
        assert [opt.state[p]["step"] for p in params] == [sum(row[k] for row in present) for k in range(4)]
    for k, (a, b) in enumerate(zip(*finals)):
        assert rel(a, b) <= (2e-4 if dtypes[k] == torch.float32 else 2e-2), k
