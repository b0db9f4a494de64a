"""GPU parity of the eigenbasis (shampoo2) low-bit flow -- the per-parameter Preconditioner with
QTensorSVDFast holders and the batched ShampooBank2 -- against the CPU restatement on top of the
quantizer oracle (oracle/shampoo2_ref.py), on identical gradients, stored states and start vectors.

How close two correct implementations can be.  One statistics update is dequantize -> Bjorck step
-> rebuild -> decay + Gram matrix -> QR(L Vt^T) -> Rayleigh quotients -> re-encode V^T in 4 bits.
The Q factor (made unique by a positive diagonal of R: the oracle flips LAPACK's columns, the
Cholesky QR produces that choice by construction) is determined to about (fp32 rounding) x
cond(L Vt^T) per column; an entry then gets another code where its scaled value sits within that
distance of a decision threshold.  Re-encoding is discontinuous, so every update is compared from
the SAME stored state (the oracle's, copied into the device holders) and the budgets are per
update:
  * well-conditioned statistics (crafted gradients, cond <= ~50): all but a stated fraction of the
    codes identical, segment maxima, kept quotients, the kept set and the largest quotient equal
    to rounding;
  * Gaussian gradients (square blocks, cond ~ order^2, and rank-deficient blocks): trailing basis
    vectors are fixed by rounding noise in ANY implementation, so codes are compared on the
    leading vectors only and, for all of them, what the optimizer uses: kept quotients, largest
    quotient, the rebuilt statistic, inverse roots and preconditioned gradients.
"""
import copy

import numpy as np
import pytest
import torch

from oracle.shampoo2_ref import RefPreconditioner2

pytestmark = pytest.mark.gpu
KW = dict(stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=128, prec_bits=4, min_lowbit_size=4096, quan_blocksize=64)


def rel(a, b):
    a, b = torch.as_tensor(a).double().cpu(), torch.as_tensor(b).double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def nibbles(codes):
    c = np.asarray(codes).reshape(-1)
    return np.stack([c >> 4, c & 15], axis=1).reshape(-1)


def conditioned(shape, block, gen, low=0.5, scale=0.02):
    """A gradient whose every block x block piece has singular values spread over [low, 1] * scale * sqrt(block)."""
    m, n = shape
    out = torch.empty(m, n)
    for r in range(0, m, block):
        for c in range(0, n, block):
            u, _ = torch.linalg.qr(torch.randn(block, block, generator=gen))
            v, _ = torch.linalg.qr(torch.randn(block, block, generator=gen))
            s = (low + (1 - low) * torch.rand(block, generator=gen)) * scale * block ** 0.5
            out[r:r + block, c:c + block] = (u * s) @ v.T
    return out


@pytest.fixture(scope="module")
def mods():
    import qtensor.functional as F
    from optimizers import shampoo2 as S2
    from optimizers import engine2 as E2
    assert torch.cuda.is_available() and F.lib is not None
    return S2, E2


class Trio:
    """The oracle, the per-parameter device path and the bank over the same parameters."""

    def __init__(self, mods, code, shapes, mode, kw):
        S2, E2 = mods
        self.shapes, self.mode = shapes, mode
        self.refs = [RefPreconditioner2(s, code, inv_root_mode=mode, positive_r=True, **kw) for s in shapes]
        qmap = {"linear-2": torch.from_numpy(code)}
        params = [torch.zeros(s, device="cuda") for s in shapes]
        self.pres = [S2.Preconditioner(p, qmap, inv_root_mode=mode, **kw) for p in params]
        self.bank = E2.ShampooBank2(params, qmap, "linear-2", inv_root_mode=mode, **kw)
        self.table = self.bank.block_table()

    def adopt_oracle_state(self):
        """Both device paths continue from the oracle's stored bits."""
        bank = self.bank
        for (pi, j, side, order, row) in self.table:
            slot = self.refs[pi].stats[2 * j + side]
            codes, absmax = (torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in slot.codes())
            h = self.pres[pi].statistics[2 * j + side]
            h.var.copy_(codes), h.absmax.copy_(absmax)
            h.Svalue, h.keep_indices, h.max_eigenvalue = slot.svalue.cuda(), slot.keep.cuda(), slot.max_eig.cuda()
            bank.basis[order].codes[row].copy_(codes), bank.basis[order].absmax[row].copy_(absmax)
            bank.svalue[order][row].copy_(slot.svalue), bank.keep[order][row].copy_(slot.keep)
            bank.max_eig[order][row].copy_(slot.max_eig)

    def update(self, grads):
        for ref, g in zip(self.refs, grads):
            ref.add_statistics(g)
        dev = [g.cuda().contiguous() for g in grads]
        for pre, g in zip(self.pres, dev):
            pre.add_statistics(g)
        self.bank.add_statistics(dev)
        torch.cuda.synchronize()

    def device_states(self, pi, j, side, order, row):
        """(name, codes, absmax, svalue, keep, max_eig, rebuilt statistic) of the two device paths."""
        h = self.pres[pi].statistics[2 * j + side]
        bank = self.bank
        rebuilt = bank._statistic(order, bank._rectified_basis(order))[row]
        yield ("per-parameter", h.var.cpu().numpy(), h.absmax.cpu(), h.Svalue.cpu(), h.keep_indices.cpu(),
               h.max_eigenvalue.cpu(), h.dequantize()[0].cpu())
        yield ("bank", bank.basis[order].codes[row].cpu().numpy(), bank.basis[order].absmax[row].cpu(),
               bank.svalue[order][row].cpu(), bank.keep[order][row].cpu(), bank.max_eig[order][row].cpu(), rebuilt.cpu())

    def roots_and_directions(self, grads, seed):
        gen = torch.Generator().manual_seed(seed)
        v0 = {(pi, j, side): torch.rand(order, generator=gen) * 2 - 1 for (pi, j, side, order, row) in self.table}
        per_order = {}
        for (pi, j, side, order, row) in self.table:
            per_order.setdefault(order, {})[row] = v0[(pi, j, side)]
        double = copy.deepcopy(self.refs)                # the same flow with the inverse roots in float64: a yardstick
        for pi, (ref, ref64, pre) in enumerate(zip(self.refs, double, self.pres)):
            starts = [v0[(pi, k // 2, k % 2)] for k in range(len(ref.stats))]
            ref.compute_preconditioners(starts)
            ref64.root_dtype = torch.float64
            ref64.compute_preconditioners(starts)
            pre.compute_preconditioners(v0=[s.cuda() for s in starts])
        self.bank.compute_preconditioners(v0={o: torch.stack([rows[r] for r in range(len(rows))]).cuda()
                                              for o, rows in per_order.items()})
        dev = [g.cuda().contiguous() for g in grads]
        want = [ref.preconditioned_grad(g) for ref, g in zip(self.refs, grads)]
        want64 = [ref.preconditioned_grad(g) for ref, g in zip(double, grads)]
        per = [pre.preconditioned_grad(g) for pre, g in zip(self.pres, dev)]
        bank = self.bank.preconditioned_grads(dev)
        torch.cuda.synchronize()
        flips = total = 0                                # stored inverse roots: codes that differ from the oracle's
        for (pi, j, side, order, row) in self.table:
            codes = self.refs[pi].precs[2 * j + side].codes()[0]
            for got in (self.pres[pi].preconditioners[2 * j + side].var, self.bank.precs[order].codes[row]):
                flips += int(np.count_nonzero(nibbles(got.cpu().numpy()) != nibbles(codes)))
                total += order * order
        self.root_flips = flips / total
        return want, want64, per, bank


def direction_report(want, want64, per, bank):
    """Per parameter: (oracle fp32 vs float64 yardstick, device paths vs yardstick, device paths vs oracle fp32)."""
    rows = []
    for w, w64, p, b in zip(want, want64, per, bank):
        p, b = p.reshape(w.shape), b.reshape(w.shape)
        rows.append((rel(w, w64), max(rel(p, w64), rel(b, w64)), max(rel(p, w), rel(b, w))))
    return rows


@pytest.mark.parametrize("mode", [1, 0])
def test_well_conditioned_statistics_follow_the_oracle_code_for_code(mods, code_maps, mode, tmp_path, monkeypatch):
    monkeypatch.chdir(tmp_path)
    code = code_maps[("linear-2", 4)]
    shapes = [(128, 256), (256, 128), (128, 1, 128)]
    trio = Trio(mods, code, shapes, mode, KW)
    gen = torch.Generator().manual_seed(31)
    worst = dict(flips=0.0, absmax=0.0, svalue=0.0, top=0.0, keep=0, rebuilt=0.0)
    total_codes = total_flips = 0
    for st in range(3):
        grads = [conditioned((s[0], s[-1]), 128, gen).reshape(s) for s in shapes]
        trio.adopt_oracle_state()
        trio.update(grads)
        assert trio.bank.qr_fallbacks == 0
        for entry in trio.table:
            pi, j, side, order, row = entry
            slot = trio.refs[pi].stats[2 * j + side]
            codes, absmax = slot.codes()
            want_stat = slot.dequantize()[0]
            top = float(slot.max_eig)
            for name, c, a, s, k, mx, stat in trio.device_states(*entry):
                flips = int(np.count_nonzero(nibbles(c) != nibbles(codes)))
                total_flips += flips
                total_codes += order * order
                worst["flips"] = max(worst["flips"], flips / (order * order))
                worst["absmax"] = max(worst["absmax"], rel(a, absmax))
                worst["svalue"] = max(worst["svalue"], float((s - slot.svalue).abs().max()) / top)
                worst["top"] = max(worst["top"], abs(float(mx) - top) / top)
                worst["keep"] = max(worst["keep"], len(set(k.tolist()) ^ set(slot.keep.tolist())))
                worst["rebuilt"] = max(worst["rebuilt"], rel(stat, want_stat))
    print("well-conditioned, mode", mode, worst, "flips", total_flips, "of", total_codes)
    # (one differing code of an order-128 basis moves the rebuilt statistic by about 2e-3 of its norm)
    assert total_flips <= 5e-5 * total_codes and worst["flips"] <= 5e-4
    assert worst["absmax"] <= 1e-5 and worst["svalue"] <= 1e-5 and worst["top"] <= 1e-5 and worst["keep"] == 0
    assert worst["rebuilt"] <= 1e-2
    trio.adopt_oracle_state()
    rows = direction_report(*trio.roots_and_directions(grads, 77))
    print("preconditioned gradients (fp32 oracle vs float64, device vs float64, device vs fp32 oracle)", rows,
          "differing codes of the inverse roots", trio.root_flips)
    # (one differing 4-bit code in an inverse root of order 128 moves the direction by about 5e-4)
    assert trio.root_flips <= 2e-4
    # (measured: up to 2.2e-3 with four differing codes in one inverse root)
    assert all(dev <= 2 * ref + 3e-3 and direct <= 4e-3 for ref, dev, direct in rows)
    for (pi, j, side, order, row) in trio.table:
        slot = trio.refs[pi].precs[2 * j + side]
        # (a differing 4-bit code moves an inverse root of order 128 by about 6e-4 of its norm; measured up to 2.3e-3)
        assert rel(trio.pres[pi].preconditioners[2 * j + side].dequantize(), slot.get()) <= 4e-3


@pytest.mark.parametrize("mode", [1, 0])
def test_gaussian_gradients_follow_the_oracle_in_what_the_optimizer_uses(mods, code_maps, mode, tmp_path, monkeypatch):
    monkeypatch.chdir(tmp_path)
    code = code_maps[("linear-2", 4)]
    shapes = [(128, 192), (256, 128), (128, 1, 256)]             # 128 x 64 blocks give rank-deficient statistics
    trio = Trio(mods, code, shapes, mode, KW)
    gen = torch.Generator().manual_seed(21)
    worst = dict(lead=0.0, all=0.0, svalue=0.0, top=0.0, rebuilt=0.0)
    for st in range(3):
        grads = [0.02 * torch.randn(s, generator=gen) for s in shapes]
        trio.adopt_oracle_state()
        trio.update(grads)
        for entry in trio.table:
            pi, j, side, order, row = entry
            slot = trio.refs[pi].stats[2 * j + side]
            codes, absmax = slot.codes()
            want_stat = slot.dequantize()[0]
            top = float(slot.max_eig)
            lead = order * (order // 4)                              # rows of Vt = leading columns of Q
            for name, c, a, s, k, mx, stat in trio.device_states(*entry):
                differ = nibbles(c) != nibbles(codes)
                worst["lead"] = max(worst["lead"], np.count_nonzero(differ[:lead]) / lead)
                worst["all"] = max(worst["all"], np.count_nonzero(differ) / differ.size)
                worst["svalue"] = max(worst["svalue"], float((s - slot.svalue).abs().max()) / top)
                worst["top"] = max(worst["top"], abs(float(mx) - top) / top)
                worst["rebuilt"] = max(worst["rebuilt"], float((stat.double() - want_stat.double()).norm()) /
                                       max(float(want_stat.norm()), top))
    print("gaussian, mode", mode, worst)
    assert worst["lead"] <= 1e-3 and worst["svalue"] <= 1e-5 and worst["top"] <= 1e-5 and worst["rebuilt"] <= 2e-3
    trio.adopt_oracle_state()
    rows = direction_report(*trio.roots_and_directions(grads, 78))
    print("preconditioned gradients (fp32 oracle vs float64, device vs float64, device vs fp32 oracle)", rows,
          "differing codes of the inverse roots", trio.root_flips)
    assert all(dev <= 2 * ref + 2e-3 and direct <= 1e-2 for ref, dev, direct in rows)


@pytest.mark.parametrize("mode", [1, 0])
def test_vanishing_gradients_end_where_the_oracle_ends(mods, code_maps, mode, tmp_path, monkeypatch):
    """All-zero gradients: the reference's update keeps the smaller half of the Rayleigh quotients, which is the half
    the rebuilt statistic (rank n/2) does not reach -- zeros -- so after two updates the statistic is exactly zero and
    its inverse root is not finite.  The device paths must not invent anything else: same stored quotients, and
    non-finite roots where the oracle's are."""
    monkeypatch.chdir(tmp_path)
    code = code_maps[("linear-2", 4)]
    shapes = [(128, 192), (256, 128)]
    trio = Trio(mods, code, shapes, mode, KW)
    grads = [torch.zeros(s) for s in shapes]
    for st in range(3):
        trio.adopt_oracle_state()
        trio.update(grads)
    for entry in trio.table:
        pi, j, side, order, row = entry
        slot = trio.refs[pi].stats[2 * j + side]
        assert float(slot.svalue.abs().max()) == 0.0 and float(slot.max_eig) == 0.0
        for name, c, a, s, k, mx, stat in trio.device_states(*entry):
            assert float(s.abs().max()) == 0.0 and float(mx) == 0.0, name
            assert float(stat.abs().max()) == 0.0, name
    assert trio.bank.qr_fallbacks == 0
    trio.adopt_oracle_state()
    want, _, per, bank = trio.roots_and_directions(grads, 5)
    for w, p_, b in zip(want, per, bank):
        assert not bool(torch.isfinite(torch.as_tensor(w)).all())
        assert not bool(torch.isfinite(p_).all()) and not bool(torch.isfinite(b).all())

