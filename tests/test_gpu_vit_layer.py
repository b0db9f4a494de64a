"""One transformer layer of a ViT-B/32 at full size -- 768 x 2304 (qkv), 768 x 768 (proj), 768 x 3072
(fc1), 3072 x 768 (fc2), prec_maxorder 1024, so blocks of orders 768 / 1024 / 256 exactly as in the
full model (2304 -> 1024 + 1024 + 256, 3072 -> 3 x 1024) -- through the statistics update, the
coupled-Newton inverse roots and the preconditioned gradient, for both low-bit variants, on the
per-parameter device path and on the batched bank, against the CPU restatements of the reference
flow (oracle/shampoo_ref.py, oracle/shampoo2_ref.py; C form of the quantizer).

Gradients are N(0, 0.02^2) as in the benchmark.  Their statistics are not all regular: a 768 x 256 block
gives a rank-256 term in a 768 x 768 statistic.  Budgets as in the small-order tests (see
test_gpu_shampoo.py and test_gpu_shampoo2_oracle.py), per update from the same stored state for the
eigenbasis variant."""
import copy

import numpy as np
import pytest
import torch

from oracle.shampoo_ref import RefPreconditioner
from test_gpu_shampoo2_oracle import Trio, direction_report, nibbles, rel

pytestmark = pytest.mark.gpu
LAYER = [(768, 2304), (768, 768), (768, 3072), (3072, 768)]
KW = dict(stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1024, prec_bits=4, min_lowbit_size=4096, quan_blocksize=64)


@pytest.fixture(scope="module")
def layer_grads():
    gen = torch.Generator().manual_seed(2024)
    return [[0.02 * torch.randn(s, generator=gen) for s in LAYER] for _ in range(2)]


def test_naive_variant_on_one_full_size_layer(code_maps, layer_grads):
    import qtensor.functional as F
    from optimizers import shampoo1 as S1
    from optimizers.engine import ShampooBank
    assert torch.cuda.is_available() and F.lib is not None
    code = code_maps[("linear-2", 4)]
    qmap = {"linear-2": torch.from_numpy(code)}
    params = [torch.zeros(s, device="cuda") for s in LAYER]
    refs = [RefPreconditioner(s, code, **KW) for s in LAYER]
    pres = [S1.Preconditioner(p, qmap, **KW) for p in params]
    bank = ShampooBank(params, qmap, "linear-2", **KW)
    table = bank.block_table()
    assert sorted(bank.per_order.items()) == [(256, 1), (768, 11), (1024, 8)]
    for grads in layer_grads:
        dev = [g.cuda() for g in grads]
        for ref, pre, g, d in zip(refs, pres, grads, dev):
            ref.add_statistics(g)
            pre.add_statistics(d)
        bank.add_statistics(dev)
    flips = total = 0
    for (pi, j, side, order, row) in table:
        slot, h = refs[pi].stats[2 * j + side], pres[pi].statistics[2 * j + side]
        codes, absmax, diag = slot.codes()
        assert torch.equal(bank.stats[order].codes[row], h.var) and torch.equal(bank.stats[order].absmax[row], h.absmax)
        assert torch.equal(bank.stats[order].diag[row], h.diag)
        flips += int(np.count_nonzero(nibbles(h.var.cpu().numpy()) != nibbles(codes)))
        total += order * order
        assert rel(h.absmax, absmax) <= 1e-5 and rel(h.diag, diag) <= 1e-5
        assert rel(h.dequantize(), slot.get()) <= 1e-3
    print("naive variant: differing codes after two updates", flips, "of", total)
    assert flips <= 1e-4 * total
    # The inverse roots start from the SAME stored statistics (the oracle's bits): a 768 x 256 block leaves its
    # 768 x 768 statistic with a numerical null space, where one differing code moves the inverse root by far
    # more than any rounding does, in any implementation.
    for (pi, j, side, order, row) in table:
        codes, absmax, diag = (torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in refs[pi].stats[2 * j + side].codes())
        h = pres[pi].statistics[2 * j + side]
        h.var.copy_(codes), h.absmax.copy_(absmax), h.diag.copy_(diag)
        bank.stats[order].codes[row].copy_(codes), bank.stats[order].absmax[row].copy_(absmax), bank.stats[order].diag[row].copy_(diag)
    gen = torch.Generator().manual_seed(9)
    v0 = {(pi, j, side): torch.rand(order, generator=gen) * 2 - 1 for (pi, j, side, order, row) in table}
    stacked = {o: torch.empty(n, o) for o, n in bank.per_order.items()}
    for (pi, j, side, order, row) in table:
        stacked[order][row] = v0[(pi, j, side)]
    double = copy.deepcopy(refs)                          # the same flow with the Newton iteration in float64: a yardstick
    for pi, (ref, ref64, pre) in enumerate(zip(refs, double, pres)):
        starts = [v0[(pi, k // 2, k % 2)] for k in range(len(ref.stats))]
        ref.compute_preconditioners(starts)
        ref64.root_dtype = torch.float64
        ref64.compute_preconditioners(starts)
        pre.compute_preconditioners([s.cuda() for s in starts])
    bank.compute_preconditioners({o: v.cuda() for o, v in stacked.items()})
    dev = [g.cuda() for g in layer_grads[-1]]
    outs = bank.preconditioned_grads(dev)
    rows = direction_report([ref.preconditioned_grad(g) for ref, g in zip(refs, layer_grads[-1])],
                            [ref.preconditioned_grad(g) for ref, g in zip(double, layer_grads[-1])],
                            [pre.preconditioned_grad(d) for pre, d in zip(pres, dev)], outs)
    print("naive variant: preconditioned gradients (fp32 oracle vs float64, device vs float64, device vs fp32 oracle)", rows)
    flips = total = 0
    for (pi, j, side, order, row) in table:
        codes = refs[pi].precs[2 * j + side].codes()[0]
        for got in (pres[pi].preconditioners[2 * j + side].var, bank.precs[order].codes[row]):
            flips += int(np.count_nonzero(nibbles(got.cpu().numpy()) != nibbles(codes)))
            total += order * order
    print("naive variant: differing codes of the inverse roots", flips, "of", total)
    assert flips <= 1e-4 * total
    assert all(dev <= 2 * ref + 5e-4 and direct <= 1e-3 for ref, dev, direct in rows)


def test_eigenbasis_variant_on_one_full_size_layer(code_maps, layer_grads, tmp_path, monkeypatch):
    import qtensor.functional as F
    from optimizers import shampoo2 as S2
    from optimizers import engine2 as E2
    assert torch.cuda.is_available() and F.lib is not None
    monkeypatch.chdir(tmp_path)
    trio = Trio((S2, E2), code_maps[("linear-2", 4)], LAYER, 1, KW)
    assert sorted(trio.bank.per_order.items()) == [(256, 1), (768, 11), (1024, 8)]
    # regular: the smallest kept quotient is above 1e-3 of the largest one (the 768-order statistics of 768 x 1024 and
    # 768 x 768 blocks, the 256-order one); the others have a numerical null space (1024-order statistics of
    # 768 x 1024 blocks: rank 768 + the start value; the 768-order one of the 768 x 256 block: rank 256), whose
    # basis vectors rounding noise alone decides, in any implementation
    worst = {True: dict(lead=0.0, all=0.0, svalue=0.0, top=0.0, rebuilt=0.0), False: dict(lead=0.0, all=0.0, svalue=0.0, top=0.0, rebuilt=0.0)}
    seen = {True: 0, False: 0}
    for grads in layer_grads:
        trio.adopt_oracle_state()
        trio.update(grads)
        for entry in trio.table:
            pi, j, side, order, row = entry
            slot = trio.refs[pi].stats[2 * j + side]
            codes, absmax = slot.codes()
            want_stat = slot.dequantize()[0]
            top = float(slot.max_eig)
            regular = float(slot.svalue.min()) > 1e-3 * top
            seen[regular] += 1
            w = worst[regular]
            lead = order * (order // 4)                              # rows of Vt = leading columns of Q
            for name, c, a, s, k, mx, stat in trio.device_states(*entry):
                differ = nibbles(c) != nibbles(codes)
                w["lead"] = max(w["lead"], np.count_nonzero(differ[:lead]) / lead)
                w["all"] = max(w["all"], np.count_nonzero(differ) / differ.size)
                w["svalue"] = max(w["svalue"], float((s - slot.svalue).abs().max()) / top)
                w["top"] = max(w["top"], abs(float(mx) - top) / top)
                w["rebuilt"] = max(w["rebuilt"], float((stat.double() - want_stat.double()).norm()) /
                                   max(float(want_stat.norm()), top))
    print("eigenbasis variant, regular statistics:", seen[True], worst[True])
    print("eigenbasis variant, statistics with a null space:", seen[False], worst[False], "library QR fallbacks", trio.bank.qr_fallbacks)
    assert seen[True] >= 20 and seen[False] >= 10
    w = worst[True]
    assert w["all"] <= 1e-4 and w["svalue"] <= 1e-5 and w["top"] <= 1e-5 and w["rebuilt"] <= 2e-3
    w = worst[False]
    assert w["lead"] <= 1e-4 and w["svalue"] <= 1e-4 and w["top"] <= 1e-5 and w["rebuilt"] <= 5e-2
    trio.adopt_oracle_state()
    rows = direction_report(*trio.roots_and_directions(layer_grads[-1], 79))
    print("eigenbasis variant: preconditioned gradients (fp32 oracle vs float64, device vs float64, device vs fp32 oracle)", rows,
          "differing codes of the inverse roots", trio.root_flips)
    assert all(dev <= 2 * ref + 1e-3 and direct <= 1e-2 for ref, dev, direct in rows)
