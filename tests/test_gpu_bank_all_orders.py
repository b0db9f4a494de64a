"""The batched banks over every kind of block order: orders the blocksize divides (read by the products directly),
orders it does not divide (the 100 of a ViT head 768 x 100: same storage format, dequantize -> dense products ->
quantize) and orders with fewer than min_lowbit_size elements (kept in fp32, as the reference's holders keep them:
qtensor/utils.py:11-17) -- against the per-parameter device path, against the CPU restatements
(oracle/shampoo_ref.py, oracle/shampoo2_ref.py) from the same stored state, and with per-parameter selection
(`only`), which is how the fused step honours the reference's skipping of parameters without a gradient
(optimizers/shampoo2.py:415).

Budgets as in test_gpu_shampoo.py / test_gpu_shampoo2_oracle.py: a code may flip where a quotient sits within fp32
summation noise of a decision threshold (<= 1e-3 of the codes after a few updates of small matrices, <= 1e-4 at
full size from the same stored state); preconditioned gradients against the float64 yardstick of the oracle."""
import copy

import numpy as np
import pytest
import torch

from oracle.shampoo_ref import RefPreconditioner
from test_gpu_shampoo2_oracle import Trio, direction_report, nibbles, rel

pytestmark = pytest.mark.gpu
SMALL = [(128, 100), (96, 40), (128, 192), (200, 72)]         # orders 128 / 64 (flat), 100 / 96 / 72 (general layout), 40 (fp32)
KW = dict(stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=128, prec_bits=4, min_lowbit_size=4096, quan_blocksize=64)
HEAD_KW = dict(KW, prec_maxorder=1024)


def flips(got, want):
    return int(np.count_nonzero(nibbles(got.cpu().numpy()) != nibbles(want.cpu().numpy() if torch.is_tensor(want) else want)))


@pytest.fixture(scope="module")
def lib(code_maps):
    import qtensor.functional as F
    assert torch.cuda.is_available() and F.lib is not None
    return code_maps[("linear-2", 4)]


def holder_state(h):
    """(codes or the fp32 matrix, maxima, diagonal) of a per-parameter holder."""
    if h.bits >= 16:
        return h.var, None, None
    return h.var, h.absmax, getattr(h, "diag", None)


def store_row(store, row):
    import qtensor.fused as X
    if isinstance(store, X.DenseStack):
        return store.data[row], None, None
    return store.codes[row], store.absmax[row], None if store.diag is None else store.diag[row]


def test_stack_quantizer_takes_any_order(lib, code_maps):
    """quantize_stack / dequantize_stack on orders the blocksize does not divide (odd ones included: the codes of
    every matrix are padded to a whole byte) equal the single-matrix entry points, entry by entry, bit for bit."""
    import qtensor.functional as F
    import qtensor.fused as X
    g = torch.Generator().manual_seed(3)
    for bits, bs in ((4, 64), (8, 256), (4, 128)):
        code = torch.from_numpy(code_maps[("linear-2", bits)]).cuda()
        for order, batch in ((100, 3), (129, 2), (63, 4), (1, 2), (200, 1)):
            for diagreal in (False, True):
                mats = torch.randn(batch, order, order, generator=g).cuda()
                mats[0, 0, : min(order, 70)] = 0.0                          # an all-zero segment
                q = X.quantize_stack(mats, X.empty_quantized(batch, order, bs, bits, code, diagreal))
                assert not q.flat or order % bs == 0
                back = X.dequantize_stack(q)
                for b in range(batch):
                    if diagreal:
                        out, absmax, diag = F.quantize_blockwise_diagreal(mats[b].contiguous(), code, order, blocksize=bs, bits=bits)
                        want = F.dequantize_blockwise_diagreal(out, code, order, absmax, diag, blocksize=bs, bits=bits)
                        assert torch.equal(q.diag[b], diag)
                    else:
                        out, absmax = F.quantize_blockwise(mats[b].contiguous(), code, order, blocksize=bs, bits=bits)
                        want = F.dequantize_blockwise(out, code, order, absmax, blocksize=bs, bits=bits)
                    assert torch.equal(q.codes[b], out) and torch.equal(q.absmax[b], absmax)
                    assert torch.equal(back[b], want)
                    assert torch.equal(torch.signbit(back[b]), torch.signbit(want))
                # the transposed form falls back to a transposed copy for these orders
                if not diagreal:
                    qt = X.quantize_stack(mats, X.empty_quantized(batch, order, bs, bits, code, False), transposed=True)
                    for b in range(batch):
                        out, absmax = F.quantize_blockwise(mats[b].T.contiguous(), code, order, blocksize=bs, bits=bits)
                        assert torch.equal(qt.codes[b], out) and torch.equal(qt.absmax[b], absmax)
    with pytest.raises(ValueError):
        X.gemm(X.empty_quantized(1, 100, 64, 4, code, False), torch.zeros(1, 100, 8, device="cuda"))     # not readable by a product


def test_naive_bank_on_all_kinds_of_orders_equals_the_per_parameter_path(lib):
    from optimizers import shampoo1 as S1
    from optimizers.engine import ShampooBank
    import qtensor.fused as X
    code = lib
    qmap = {"linear-2": torch.from_numpy(code)}
    params = [torch.zeros(s, device="cuda") for s in SMALL]
    bank = ShampooBank(params, qmap, "linear-2", **KW)
    pres = [S1.Preconditioner(p, qmap, **KW) for p in params]
    table = bank.block_table()
    kinds = {o: ("fp32" if isinstance(q, X.DenseStack) else "flat" if q.flat else "general") for o, q in bank.stats.items()}
    assert kinds == {128: "flat", 64: "flat", 100: "general", 96: "general", 72: "general", 40: "fp32"}
    g = torch.Generator().manual_seed(31)
    for st in range(3):
        gl = [(0.02 * torch.randn(s, generator=g)).cuda() for s in SMALL]
        bank.add_statistics(gl)
        starts = {o: torch.empty(q.batch, o) for o, q in bank.stats.items()}
        per_param = []
        for pi, pre in enumerate(pres):
            pre.add_statistics(gl[pi])
            vs = [torch.rand(h.var.shape[0] if h.bits >= 16 else h.var_order, generator=g) * 2 - 1 for h in pre.statistics]
            per_param.append(vs)
            for (tpi, j, side, order, row) in table:
                if tpi == pi:
                    starts[order][row] = vs[2 * j + side]
        bank.compute_preconditioners({o: v.cuda() for o, v in starts.items()})
        outs = bank.preconditioned_grads(gl)
        for pi, pre in enumerate(pres):
            pre.compute_preconditioners([v.cuda() for v in per_param[pi]])
            want = pre.preconditioned_grad(gl[pi])
            assert rel(outs[pi], want) <= 2e-4, (SMALL[pi], st)
    differing = total = 0
    for (pi, j, side, order, row) in table:
        for store, holder in ((bank.stats[order], pres[pi].statistics[2 * j + side]), (bank.precs[order], pres[pi].preconditioners[2 * j + side])):
            got, want = store_row(store, row), holder_state(holder)
            if kinds[order] == "fp32":
                assert rel(got[0], want[0]) <= 1e-4
                continue
            # the per-parameter path multiplies these orders with the vendor's routine and adds in separate passes:
            # agreement to rounding, hence to a few codes
            differing += flips(got[0], want[0])
            total += order * order
            assert rel(got[1], want[1]) <= 1e-5 and rel(got[2], want[2]) <= 1e-5
    print("naive bank against the per-parameter path: differing codes", differing, "of", total)
    assert differing <= 1e-3 * total
    sd = bank.state_dict()
    assert "stats.40.dense" in sd and "stats.100.codes" in sd and sd["stats.100.absmax"].shape[1] == 200
    again = ShampooBank(params, qmap, "linear-2", **KW)
    again.load_state_dict(sd)
    assert all(torch.equal(a, b) for a, b in zip(again.preconditioned_grads(gl), outs))


@pytest.mark.parametrize("variant", ["shampoo1", "shampoo2"])
def test_updating_a_subset_of_the_parameters_touches_only_their_rows(lib, variant, tmp_path, monkeypatch):
    """`only`: the rows of the chosen parameters end in exactly the bits that an update of all parameters gives them,
    and every other row keeps its bits -- for the statistics, the inverse roots and the preconditioned gradients."""
    from optimizers.engine import ShampooBank
    from optimizers.engine2 import ShampooBank2
    monkeypatch.chdir(tmp_path)
    qmap = {"linear-2": torch.from_numpy(lib)}
    shapes = SMALL + [(128, 128)]
    params = [torch.zeros(s, device="cuda") for s in shapes]
    make = (lambda: ShampooBank(params, qmap, "linear-2", **KW)) if variant == "shampoo1" else \
           (lambda: ShampooBank2(params, qmap, "linear-2", inv_root_mode=1, **KW))
    g = torch.Generator().manual_seed(41)
    warm = [[(0.02 * torch.randn(s, generator=g)).cuda() for s in shapes] for _ in range(2)]
    new = [(0.02 * torch.randn(s, generator=g)).cuda() for s in shapes]
    some, everyone = make(), make()
    for bank in (some, everyone):
        for gl in warm:
            bank.add_statistics(gl)
    chosen = {0, 2}
    before = {k: v.clone() for k, v in some.state_dict().items()}
    table = some.block_table()
    starts = {o: (torch.rand(n, o, generator=g) * 2 - 1).cuda() for o, n in some.per_order.items()}
    partial = [gr if pi in chosen else None for pi, gr in enumerate(new)]
    some.add_statistics(partial, only=chosen)
    everyone.add_statistics(new)
    some.compute_preconditioners({o: v.clone() for o, v in starts.items()}, only=chosen)
    everyone.compute_preconditioners({o: v.clone() for o, v in starts.items()})
    assert some.active == [pi in chosen for pi in range(len(shapes))] and not some.is_active() and everyone.is_active()
    got, want = some.state_dict(), everyone.state_dict()
    rows_of = {}
    for (pi, j, side, order, row) in table:
        rows_of.setdefault(order, {})[row] = pi in chosen
    for name, tensor in got.items():
        parts = name.split(".")
        if len(parts) != 3 or not parts[1].isdigit():
            continue
        for row, is_chosen in rows_of[int(parts[1])].items():
            other = want[name][row] if is_chosen else before[name][row]
            assert torch.equal(tensor[row], other), (name, row, is_chosen)
    outs = some.preconditioned_grads(partial, only=chosen)
    full = everyone.preconditioned_grads(new)
    for pi in range(len(shapes)):
        assert (outs[pi] is None) == (pi not in chosen)
        if pi in chosen:
            assert torch.equal(outs[pi], full[pi])
    with pytest.raises(ValueError):
        some.add_statistics(partial, only={0, 1})                              # parameter 1 takes part and has no gradient


def test_head_768x100_through_the_naive_bank_follows_the_oracle(lib):
    """The ViT-B/32 head at full size (orders 768 and 100) through the bank: two updates against the CPU restatement,
    then inverse roots and the preconditioned gradient from the oracle's stored statistics."""
    from optimizers.engine import ShampooBank
    code = lib
    shape = (768, 100)
    qmap = {"linear-2": torch.from_numpy(code)}
    bank = ShampooBank([torch.zeros(shape, device="cuda")], qmap, "linear-2", **HEAD_KW)
    ref = RefPreconditioner(shape, code, **HEAD_KW)
    assert sorted(bank.per_order.items()) == [(100, 1), (768, 1)] and not bank.stats[100].flat and bank.stats[768].flat
    gen = torch.Generator().manual_seed(77)
    grads = [0.02 * torch.randn(shape, generator=gen) for _ in range(2)]
    for gr in grads:
        ref.add_statistics(gr)
        bank.add_statistics([gr.cuda()])
    differing = total = 0
    for (pi, j, side, order, row) in bank.block_table():
        codes, absmax, diag = ref.stats[2 * j + side].codes()
        differing += flips(bank.stats[order].codes[row], codes)
        total += order * order
        assert rel(bank.stats[order].absmax[row], absmax) <= 1e-5 and rel(bank.stats[order].diag[row], diag) <= 1e-5
    print("head through the naive bank: differing codes after two updates", differing, "of", total)
    assert differing <= 1e-4 * total
    for (pi, j, side, order, row) in bank.block_table():                      # go on from the oracle's bits
        codes, absmax, diag = (torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in ref.stats[2 * j + side].codes())
        bank.stats[order].codes[row].copy_(codes), bank.stats[order].absmax[row].copy_(absmax), bank.stats[order].diag[row].copy_(diag)
    starts = [torch.rand(o, generator=gen) * 2 - 1 for o in (768, 100)]
    ref64 = copy.deepcopy(ref)
    ref64.root_dtype = torch.float64
    ref.compute_preconditioners(starts)
    ref64.compute_preconditioners(starts)
    bank.compute_preconditioners({768: starts[0].cuda().unsqueeze(0), 100: starts[1].cuda().unsqueeze(0)})
    out = bank.preconditioned_grads([grads[-1].cuda()])[0]
    want, want64 = ref.preconditioned_grad(grads[-1]), ref64.preconditioned_grad(grads[-1])
    oracle_err, device_err = rel(want, want64), rel(out, want64)
    print("head through the naive bank: preconditioned gradient, fp32 oracle vs float64", oracle_err, "device vs float64", device_err)
    assert device_err <= 2 * oracle_err + 5e-4


def test_head_768x100_through_the_eigenbasis_bank_follows_the_oracle(lib, tmp_path, monkeypatch):
    """The same head through the eigenbasis bank (and the per-parameter device path), per update from the oracle's
    stored state: the 768-order statistic of a 768 x 100 gradient has rank 100 plus the kept half, so it is held to
    the budgets of the statistics with a null space; the 100-order one is regular."""
    import qtensor.functional as F
    from optimizers import shampoo2 as S2
    from optimizers import engine2 as E2
    assert F.lib is not None
    monkeypatch.chdir(tmp_path)
    trio = Trio((S2, E2), lib, [(768, 100)], 1, HEAD_KW)
    assert sorted(trio.bank.per_order.items()) == [(100, 1), (768, 1)]
    gen = torch.Generator().manual_seed(78)
    grads = [[0.02 * torch.randn(768, 100, generator=gen)] for _ in range(2)]
    for step in grads:
        trio.adopt_oracle_state()
        trio.update(step)
        for entry in trio.table:
            pi, j, side, order, row = entry
            slot = trio.refs[pi].stats[2 * j + side]
            codes, absmax = slot.codes()
            want_stat = slot.dequantize()[0]
            top = float(slot.max_eig)
            regular = float(slot.svalue.min()) > 1e-3 * top
            # rows of Vt = leading columns of Q; the 768-order statistic has rank 100 plus its start value, and what
            # comes after its leading 100 vectors is fixed by rounding noise in any implementation
            lead = order * min(order // 4, 64)
            for name, c, a, s, k, mx, stat in trio.device_states(*entry):
                differ = nibbles(c) != nibbles(codes)
                rebuilt = float((stat.double() - want_stat.double()).norm()) / max(float(want_stat.norm()), top)
                print(order, name, "regular" if regular else "null space", "differing codes", np.count_nonzero(differ) / differ.size,
                      "leading", np.count_nonzero(differ[:lead]) / lead, "rebuilt", rebuilt)
                assert abs(float(mx) - top) / top <= 1e-5
                assert float((s - slot.svalue).abs().max()) / top <= (1e-5 if regular else 1e-4)
                assert rebuilt <= (2e-3 if regular else 5e-2)
                assert np.count_nonzero(differ[:lead]) / lead <= (1e-3 if regular else 1e-3)
    trio.adopt_oracle_state()
    rows = direction_report(*trio.roots_and_directions(grads[-1], 80))
    print("head through the eigenbasis paths: preconditioned gradients", rows, "differing codes of the inverse roots", trio.root_flips)
    assert all(dev <= 2 * ref + 1e-3 and direct <= 1e-2 for ref, dev, direct in rows)
    assert trio.bank.qr_fallbacks == 0


@pytest.mark.parametrize("variant", ["shampoo1", "shampoo2"])
def test_full_vit_b32_step_properties(variant, tmp_path, monkeypatch):
    """All 50 parameters of the ViT-B/32 configuration (12 x {768x2304, 768x768, 768x3072, 3072x768} + 3072x768 +
    768x100) through eleven fused steps with the benchmark's settings (statistics every step, inverse roots every
    tenth): no parameter keeps a per-parameter preconditioner object, everything stays finite, a step of plain SGD
    with lr 1 moves every parameter by exactly the norm of its gradient once the preconditioners are in use (the
    preconditioned direction is rescaled to the gradient's norm), and a run resumed from a checkpoint that was read
    back with weights_only=True continues bit for bit."""
    import importlib
    import io
    monkeypatch.chdir(tmp_path)
    S = importlib.import_module("optimizers." + variant)
    shapes = [s for _ in range(12) for s in ((768, 2304), (768, 768), (768, 3072), (3072, 768))] + [(3072, 768), (768, 100)]
    kw = dict(lr=1.0, momentum=0.0, weight_decay=0.0, start_prec_step=1, stat_compute_steps=1, prec_compute_steps=10,
              stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1024, prec_bits=4, min_lowbit_size=4096, quan_blocksize=64, fused=True)
    if variant == "shampoo2":
        kw["inv_root_mode"] = 1
    torch.manual_seed(123)
    gen = torch.Generator(device="cuda").manual_seed(5)
    init = [0.02 * torch.randn(s, device="cuda", generator=gen) for s in shapes]
    grad_sets = [[0.02 * torch.randn(s, device="cuda", generator=gen) for s in shapes] for _ in range(2)]

    def run(opt, params, steps, check=False):
        for st in steps:
            for p, gr in zip(params, grad_sets[st % 2]):
                p.grad = gr.clone()
            before = [p.detach().clone() for p in params] if check and st >= 10 else None
            opt.step()
            if before is not None:
                moved = torch.stack([(p.detach() - b).norm() for p, b in zip(params, before)])
                norms = torch.stack([gr.norm() for gr in grad_sets[st % 2]])
                assert float(((moved - norms).abs() / norms).max()) <= 1e-4
        torch.cuda.synchronize()

    straight = [torch.nn.Parameter(t.clone()) for t in init]
    opt = S.ShampooSGD(straight, **kw)
    torch.manual_seed(7)
    run(opt, straight, range(6), check=True)
    sd = opt.state_dict()
    assert not any("preconditioner" in opt.state[p] for p in straight) and sd["shampoo_preconditioners"] == {}
    bank = next(iter(opt._fused_cache.values()))["bank"]
    assert len(bank.params) == 50 and sorted(bank.per_order.items()) == [(100, 1), (256, 12), (768, 136), (1024, 99)]
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    loaded = torch.load(buf, weights_only=True, map_location="cpu")
    at_six = [p.detach().clone() for p in straight]         # (parameters travel with the model's own checkpoint)
    rng = torch.cuda.get_rng_state()                        # the inverse roots of step 10 draw their start vectors
    run(opt, straight, range(6, 11), check=True)
    assert all(bool(torch.isfinite(p).all()) for p in straight)
    assert all(bank.active)

    resumed = [torch.nn.Parameter(t) for t in at_six]
    opt2 = S.ShampooSGD(resumed, **kw)
    opt2.load_state_dict(loaded)
    torch.cuda.set_rng_state(rng)
    run(opt2, resumed, range(6, 11))
    for a, b in zip(straight, resumed):
        assert torch.equal(a.detach(), b.detach())
