"""Seeded random sweeps over shapes, formats and special values: the device quantizer against the C checker bit for bit,
the stack entry points against the single-matrix ones, products against float64 (plain, transposed, skipped,
triangular, strided, pointer lists, quantized operands and addends, the requantizing and the Newton epilogue), the
orthonormalisation over ranks, conditioning and padded orders, the batched inverse roots against float64 and the CPU
form, and fused optimizer runs resumed from a checkpoint.  Each sweep is some hundreds to a thousand cases from a fixed seed; the
same drivers, left running for minutes with other seeds, are how the corner cases the other test files pin down one
by one were looked for."""
import copy
import importlib
import io
import random

import numpy as np
import pytest
import torch

from oracle import quant_np as Q

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import qtensor.functional as F
    import qtensor.fused as X
    assert torch.cuda.is_available() and F.lib is not None
    codes = {("linear", 4): Q.linear_map(True, 4, 2), ("linear", 8): Q.linear_map(True, 8, 2),
             ("dynamic", 4): Q.dynamic_map(True, 4), ("dynamic", 8): Q.dynamic_map(True, 8)}
    return F, X, {k: v.astype(np.float32) for k, v in codes.items()}


def rel(a, b):
    return float((a.double().cpu() - b.cpu()).norm() / max(float(b.norm()), 1e-30))


def bits_of(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32)).view(np.uint32).ravel()


def test_quantizer_against_the_checker(env):
    F, X, codes = env
    rnd = random.Random(1)
    for case in range(1200):
        bits = rnd.choice([4, 8]); kind = rnd.choice(["linear", "dynamic"]); bs = rnd.choice([64, 128, 256, 512, 1024, 2048])
        order = rnd.choice([1, 2, 3, 5, 17, 63, 64, 65, 100, 127, 128, 129, 169, 255, 256, 257, 300, 511, 512, 640, 777])
        diag = rnd.random() < 0.5
        dtype = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
        code = codes[(kind, bits)]
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        A = torch.randn(order, order, generator=g) * float(10.0 ** rnd.uniform(-6, 6))
        mode = rnd.choice(["plain", "outliers", "zeros", "codes", "ties", "tiny", "nan"])
        flat = A.view(-1)
        if mode == "outliers":
            flat[torch.randint(0, flat.numel(), (max(1, flat.numel() // 100),), generator=g)] *= 100
        elif mode == "zeros":
            flat[: min(flat.numel(), 3 * bs)] = 0
        elif mode == "codes":                                              # exact entries of the table times a maximum
            seg = min(bs, flat.numel())
            vals = torch.from_numpy(code)[torch.randint(0, len(code), (seg,), generator=g)] * 3.0
            vals[0] = 3.0
            flat[:seg] = vals
        elif mode == "ties":                                               # midpoints between neighbouring entries
            srt = np.sort(code)
            mid = torch.from_numpy(((srt[1:].astype(np.float64) + srt[:-1]) / 2).astype(np.float32))
            seg = min(bs, flat.numel())
            vals = mid[torch.randint(0, len(mid), (seg,), generator=g)] * 2.0
            vals[0] = 2.0
            flat[:seg] = vals
        elif mode == "tiny":
            flat[: min(flat.numel(), bs)] *= 1e-38
        elif mode == "nan" and flat.numel() > 3:
            flat[3] = float("nan")
        A = A.to(dtype)
        code_d = torch.from_numpy(code).cuda()
        if diag:
            out, absmax, dg = F.quantize_blockwise_diagreal(A.cuda(), code_d, order, blocksize=bs, bits=bits)
            back = F.dequantize_blockwise_diagreal(out, code_d, order, absmax, dg, blocksize=bs, bits=bits)
        else:
            out, absmax = F.quantize_blockwise(A.cuda(), code_d, order, blocksize=bs, bits=bits)
            dg = None
            back = F.dequantize_blockwise(out, code_d, order, absmax, blocksize=bs, bits=bits)
        ref = Q.quantize_c(A.float().numpy(), code, order, bs, bits, store_diag=diag)
        want = np.asarray(Q.dequantize_c(ref[0], code, order, ref[1], bs, bits, diag=ref[2] if diag else None), dtype=np.float32).ravel()
        tag = (case, bits, kind, bs, order, diag, str(dtype), mode)
        assert np.array_equal(out.cpu().numpy().ravel(), np.asarray(ref[0]).ravel()), tag
        assert np.array_equal(bits_of(absmax.cpu().numpy()), bits_of(ref[1])), tag
        if diag:
            assert np.array_equal(bits_of(dg.cpu().numpy()), bits_of(ref[2])), tag
        got = back.float().cpu().numpy().ravel()
        nan = np.isnan(want)
        assert np.array_equal(bits_of(got[~nan]), bits_of(want[~nan])) and np.isnan(got[nan]).all(), tag


def test_stack_entry_points_against_the_single_matrix_ones(env):
    F, X, codes = env
    rnd = random.Random(2)
    dev_codes = {b: torch.from_numpy(codes[("linear", b)]).cuda() for b in (4, 8)}
    for case in range(250):
        bits = rnd.choice([4, 8]); bs = rnd.choice([64, 128, 256])
        order = rnd.choice([1, 3, 17, 63, 64, 65, 100, 128, 129, 192, 200, 256, 300, 320, 512])
        batch = rnd.choice([1, 2, 3, 7, 16])
        diag = rnd.random() < 0.5
        transposed = rnd.random() < 0.4 and not diag
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        mats = (torch.randn(batch, order, order, generator=g) * float(10.0 ** rnd.uniform(-4, 4))).cuda()
        if rnd.random() < 0.3:
            mats[0].view(-1)[: min(order * order, 2 * bs)] = 0
        code = dev_codes[bits]
        q = X.quantize_stack(mats, X.empty_quantized(batch, order, bs, bits, code, diag), transposed=transposed)
        back = X.dequantize_stack(q)
        tag = (case, bits, bs, order, batch, diag, transposed)
        for b in range(batch):
            src = mats[b].T.contiguous() if transposed else mats[b].contiguous()
            if diag:
                out, absmax, dg = F.quantize_blockwise_diagreal(src, code, order, blocksize=bs, bits=bits)
                want = F.dequantize_blockwise_diagreal(out, code, order, absmax, dg, blocksize=bs, bits=bits)
                assert torch.equal(q.diag[b], dg), tag
            else:
                out, absmax = F.quantize_blockwise(src, code, order, blocksize=bs, bits=bits)
                want = F.dequantize_blockwise(out, code, order, absmax, blocksize=bs, bits=bits)
            assert torch.equal(q.codes[b].view(-1), out.view(-1)) and torch.equal(q.absmax[b].view(-1), absmax.view(-1)), tag
            assert torch.equal(back[b], want), tag
        if batch >= 3:
            sub = X.dequantize_stack(q.select(torch.tensor([batch - 1, 0], device="cuda")))
            assert torch.equal(sub[0], back[batch - 1]) and torch.equal(sub[1], back[0]), tag


DIMS = [1, 2, 3, 5, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 384, 512, 640, 1000]


def test_products_against_float64(env):
    F, X, codes = env
    rnd = random.Random(3)
    dev_codes = {b: torch.from_numpy(codes[("linear", b)]).cuda() for b in (4, 8)}
    for case in range(1500):
        batch = rnd.choice([1, 1, 2, 3, 5, 9])
        pipe = rnd.choice([None, "f32", "split"])
        kind = rnd.choice(["dense", "dense", "quantA", "quantB", "sym", "addend", "skip", "skip", "upper", "upper_b", "strided", "ptrlist"])
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        tag = [case, kind, batch, pipe]
        if kind in ("quantA", "quantB"):
            order = rnd.choice([64, 128, 192, 256, 320, 512]); other = rnd.choice(DIMS); bits = rnd.choice([4, 8])
            bs = rnd.choice([64, 128, 256])
            if order % bs:
                bs = 64
            q = X.quantize_stack(torch.randn(batch, order, order, generator=g).cuda(),
                                 X.empty_quantized(batch, order, bs, bits, dev_codes[bits], rnd.random() < 0.5))
            deq = X.dequantize_stack(q).double().cpu()
            tag += [order, other, bits, bs]
            if kind == "quantA":
                B = torch.randn(batch, order, other, generator=g).cuda()
                got, want = X.gemm(q, B, pipe=pipe), deq @ B.double().cpu()
            else:
                A = torch.randn(batch, other, order, generator=g).cuda()
                got, want = X.gemm(A, q, pipe=pipe), A.double().cpu() @ deq
        elif kind == "ptrlist":
            m, n, k = rnd.choice(DIMS), rnd.choice(DIMS), rnd.choice(DIMS)
            pa, pb, pc = (torch.randn(batch + 2, m, k, generator=g).cuda(), torch.randn(batch + 2, k, n, generator=g).cuda(),
                          torch.zeros(batch + 2, m, n, device="cuda"))
            ia = [rnd.randrange(batch + 2) for _ in range(batch)]; ib = [rnd.randrange(batch + 2) for _ in range(batch)]
            ic = rnd.sample(range(batch + 2), batch)
            table = lambda pool, idx: torch.tensor([pool[i].data_ptr() for i in idx], dtype=torch.int64).cuda()      # noqa: E731
            X.gemm(X.PtrList(table(pa, ia), (batch, m, k)), X.PtrList(table(pb, ib), (batch, k, n)),
                   out=X.PtrList(table(pc, ic), (batch, m, n)), pipe=pipe)
            got = torch.stack([pc[i] for i in ic])
            want = torch.stack([pa[i].double().cpu() @ pb[j].double().cpu() for i, j in zip(ia, ib)])
            tag += [m, n, k]
        else:
            m, n, k = rnd.choice(DIMS), rnd.choice(DIMS), rnd.choice(DIMS)
            ta, tb = rnd.random() < 0.4, rnd.random() < 0.4
            if ta and tb:
                tb = False                                                 # (A^T B^T is not built: it is (B A)^T)
            if kind == "sym":
                n = m
                ta, tb = (False, True) if rnd.random() < 0.5 else (True, False)
            if kind in ("upper", "upper_b", "strided"):
                ta = tb = False
            if kind == "upper":
                k = m
            if kind == "upper_b":
                k = n
            pad = rnd.choice([0, 4, 7, 64]) if kind == "strided" else 0
            A = torch.randn((batch, k, m) if ta else (batch, m, k + pad), generator=g).cuda()
            B = torch.randn((batch, n, k) if tb else (batch, k, n + pad), generator=g).cuda()
            if pad:
                A, B = A[:, :, :k], B[:, :, :n]
            if kind == "upper":
                A = torch.triu(A)
            if kind == "upper_b":
                B = torch.triu(B)
            Ad = (A.transpose(1, 2) if ta else A).double().cpu()
            Bd = (B.transpose(1, 2) if tb else B).double().cpu()
            tag += [m, n, k, ta, tb, pad]
            if kind == "sym":
                got, want = X.gemm(A, A, trans_a=ta, trans_b=tb, symmetric=True, pipe=pipe), Ad @ Ad.transpose(1, 2)
                assert torch.equal(got, got.transpose(1, 2)), tag
            elif kind == "addend":
                E = torch.randn(batch, m, n, generator=g).cuda()
                al, be = rnd.uniform(-2, 2), rnd.uniform(-2, 2)
                got = X.gemm(A, B, trans_a=ta, trans_b=tb, addend=E, alpha=al, beta=be, pipe=pipe)
                want = al * (Ad @ Bd) + be * E.double().cpu()
            elif kind == "skip":
                skip = torch.tensor([rnd.randint(0, 1) for _ in range(batch)], dtype=torch.int32).cuda()
                got = X.gemm(A, B, trans_a=ta, trans_b=tb, out=torch.full((batch, m, n), 7.0, device="cuda"), skip=skip, pipe=pipe)
                want = Ad @ Bd
                want[skip.cpu().bool()] = 7.0
            elif kind == "strided":
                whole = torch.zeros(batch, m, n + pad, device="cuda")
                got = X.gemm(A, B, out=whole[:, :, :n], pipe=pipe)
                want = Ad @ Bd
                assert pad == 0 or bool((whole[:, :, n:] == 0).all()), tag
            else:
                got = X.gemm(A, B, trans_a=ta, trans_b=tb, upper_a=kind == "upper", upper_b=kind == "upper_b", pipe=pipe)
                want = Ad @ Bd
        assert tuple(got.shape) == tuple(want.shape) and rel(got, want) <= 2e-5, tag


def test_special_epilogues(env):
    F, X, codes = env
    rnd = random.Random(4)
    dev_codes = {b: torch.from_numpy(codes[("linear", b)]).cuda() for b in (4, 8)}

    def duplicate(q):
        c = copy.copy(q)
        c.codes, c.absmax = q.codes.clone(), q.absmax.clone()
        c.diag = None if q.diag is None else q.diag.clone()
        return c

    for case in range(600):
        batch = rnd.choice([1, 2, 3, 5]); pipe = rnd.choice([None, "f32", "split"])
        kind = rnd.choice(["axpbyq", "requant", "newton"])
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        tag = [case, kind, batch, pipe]
        if kind == "newton":
            m = rnd.choice([64, 100, 128, 200, 256, 320])
            A = torch.randn(batch, m, m, generator=g).cuda() / m ** 0.5
            B = torch.randn(batch, m, m, generator=g).cuda() / m ** 0.5
            sym = rnd.random() < 0.5
            if sym:
                A = (A + A.transpose(1, 2)).contiguous()
                B = A
            w = rnd.uniform(-1, 1)
            C, T, err = torch.empty(batch, m, m, device="cuda"), torch.empty(batch, m, m, device="cuda"), torch.zeros(batch, device="cuda")
            X.gemm(A, B, out=C, newton=(T, w, err), symmetric=sym, pipe=pipe)
            P = A.double().cpu() @ B.double().cpu()
            eye = torch.eye(m, dtype=torch.float64)
            far = (P - eye).abs().amax(dim=(1, 2))
            assert rel(C, P) <= 2e-5 and rel(T, (1 - w) * eye + w * P) <= 2e-5, tag + [m, sym]
            assert float(((err.double().cpu() - far).abs() / far).max()) <= 1e-4, tag + [m, sym]
            continue
        order = rnd.choice([64, 128, 192, 256, 320, 512]); k = rnd.choice(DIMS); bits = rnd.choice([4, 8])
        bs = 64 if kind == "requant" else rnd.choice([64, 128])
        if order % bs:
            bs = 64
        diag = rnd.random() < 0.5
        left = rnd.random() < 0.5                                          # G G^T or G^T G
        G = torch.randn((batch, order, k) if left else (batch, k, order), generator=g).cuda()
        E = torch.randn(batch, order, order, generator=g)
        q = X.quantize_stack((E + E.transpose(1, 2)).cuda(), X.empty_quantized(batch, order, bs, bits, dev_codes[bits], diag))
        al, be = rnd.uniform(0.01, 1), rnd.uniform(0.5, 1)
        tag += [order, k, bits, bs, diag, left]
        fp = X.gemm(G, G, trans_a=not left, trans_b=left, addend=q, alpha=al, beta=be, pipe=pipe)
        if kind == "axpbyq":
            Gd = G.double().cpu()
            prod = Gd @ Gd.transpose(1, 2) if left else Gd.transpose(1, 2) @ Gd
            assert rel(fp, be * X.dequantize_stack(q).double().cpu() + al * prod) <= 2e-5, tag
        else:                                                              # the same bits as product, then quantizer
            two = X.quantize_stack(fp, X.empty_quantized(batch, order, bs, bits, dev_codes[bits], diag))
            one = X.gemm(G, G, trans_a=not left, trans_b=left, addend=duplicate(q), alpha=al, beta=be, requantize=True, pipe=pipe)
            assert torch.equal(one.codes, two.codes) and torch.equal(one.absmax, two.absmax), tag
            assert not diag or torch.equal(one.diag, two.diag), tag


def test_orthonormal_bases_of_all_kinds_of_stacks(env):
    F, X, codes = env
    rnd = random.Random(11)
    for case in range(400):
        n = rnd.choice([1, 2, 7, 40, 63, 64, 65, 100, 128, 130, 192, 200, 256, 300, 384])
        B = rnd.choice([1, 2, 3, 6, 17])
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        mats, kinds = [], []
        for b in range(B):
            kind = rnd.choice(["plain", "cond", "graded", "repeat", "lowrank", "lowrank_noise", "zero_cols", "subspace"])
            if kind == "plain" or n < 4:
                Y = torch.randn(n, n, generator=g)
            elif kind == "cond":
                u, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
                v, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
                Y = ((u * torch.logspace(0, -rnd.uniform(0, 8), n, dtype=torch.float64)) @ v.T).float()
            elif kind == "graded":
                Y = torch.randn(n, n, generator=g) * torch.logspace(0, -rnd.uniform(0, 12), n)
            elif kind == "repeat":
                Y = torch.randn(n, n, generator=g)
                j = rnd.randrange(1, n)
                Y[:, j] = Y[:, rnd.randrange(0, j)] * rnd.uniform(0.5, 2)
            elif kind in ("lowrank", "lowrank_noise"):
                r = rnd.randrange(1, n)
                Y = torch.randn(n, r, generator=g) @ torch.randn(r, n, generator=g)
                if kind == "lowrank_noise":
                    Y = Y + 1e-7 * torch.randn(n, n, generator=g)
            elif kind == "zero_cols":
                Y = torch.randn(n, n, generator=g)
                Y[:, rnd.randrange(n)] = 0
            else:                                                          # one step of subspace iteration: L V with V nearly orthonormal
                u, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
                L = (u * torch.logspace(0, -rnd.uniform(0, 6), n, dtype=torch.float64)) @ u.T
                V, _ = torch.linalg.qr(u + 0.05 * torch.randn(n, n, generator=g, dtype=torch.float64))
                Y = (L @ V).float()
            mats.append(Y * float(10.0 ** rnd.uniform(-3, 3)))
            kinds.append(kind)
        Y = torch.stack(mats).cuda()
        Qm, redone = X.cholesky_qr(Y)
        gram = Qm.double().transpose(1, 2) @ Qm.double()
        off = (gram - torch.eye(n, dtype=torch.float64, device="cuda")).abs().amax(dim=(1, 2)).cpu()
        assert bool(torch.isfinite(Qm).all()) and float(off.max()) <= 5e-5, (case, n, B, kinds, off.tolist())
        for b, kind in enumerate(kinds):
            if kind == "plain" and n >= 8:                                 # nested spans where they are well defined
                lead = Y[b, :, : n // 2].double()
                proj = Qm[b, :, : n // 2].double() @ (Qm[b, :, : n // 2].double().T @ lead)
                assert float((proj - lead).norm() / lead.norm()) <= 1e-4, (case, n, b)


def test_inverse_roots_of_random_spectra(env):
    from optimizers import matrix_functions as MF
    rnd = random.Random(3)
    for case in range(60):
        n = rnd.choice([2, 3, 7, 33, 64, 65, 100, 128, 130, 200, 256]); B = rnd.choice([1, 2, 3, 5]); p = rnd.choice([2, 4, 4, 8])
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        mats = []
        for b in range(B):
            u, _ = torch.linalg.qr(torch.randn(n, n, generator=g, dtype=torch.float64))
            lam = torch.logspace(0, -rnd.uniform(0, 6), n, dtype=torch.float64) * float(10.0 ** rnd.uniform(-4, 2))
            if rnd.random() < 0.2:
                lam[n // 2:] = 0                                           # rank deficient: the ridge carries it
            A = (u * lam) @ u.T
            mats.append((A + A.T) / 2)
        A64 = torch.stack(mats)
        A32 = A64.float()
        symmetric = bool(torch.equal(A32, A32.transpose(1, 2))) and rnd.random() < 0.7
        v0 = torch.rand(B, n, generator=g) * 2 - 1
        got = MF.ComputePowerBatched(A32.clone().cuda(), p, ridge_epsilon=1e-6, v0=v0.cuda(), symmetric=symmetric).double().cpu()
        for b in range(B):
            lam_b, U = torch.linalg.eigh(A64[b])
            want = (U * (lam_b.clamp_min(0) + 1e-6 * float(lam_b.max())).pow(-1.0 / p)) @ U.T
            cpu = MF.ComputePower(A32[b].clone(), p, ridge_epsilon=1e-6, v0=v0[b].clone()).double()
            e_gpu, e_cpu = float((got[b] - want).norm() / want.norm()), float((cpu - want).norm() / want.norm())
            assert bool(torch.isfinite(got[b]).all()) and e_gpu <= 2 * e_cpu + 1e-4, (case, n, B, p, symmetric, b, e_gpu, e_cpu)


POOL = [(64, 64), (130, 65), (300, 20), (257, 129), (7, 300), (100, 100), (96, 40), (128, 192), (200, 72), (1, 80), (512, 33),
        (65, 64), (3, 5), (256, 256), (24, 24, 3), (50,)]


@pytest.mark.parametrize("variant", ["shampoo1", "shampoo2"])
def test_fused_runs_resume_bit_for_bit(variant, tmp_path, monkeypatch):
    """Random parameter sets (matrices of all kinds of shapes, a convolution weight, a vector), settings and missing
    gradients: a fused run that is saved at a random step, read back with weights_only=True into a fresh optimizer and
    continued ends with the same bits as the run that was never interrupted."""
    monkeypatch.chdir(tmp_path)
    S = importlib.import_module("optimizers." + variant)
    for seed in range(12):
        rnd = random.Random(seed)
        shapes = rnd.sample(POOL, rnd.randint(2, 6))
        kw = dict(lr=1e-2, weight_decay=0.01, start_prec_step=rnd.choice([1, 2, 4]), stat_compute_steps=rnd.choice([1, 2]),
                  prec_compute_steps=rnd.choice([2, 3, 4]), stat_decay=0.95, matrix_eps=1e-6,
                  prec_maxorder=rnd.choice([64, 100, 128, 256]), prec_bits=rnd.choice([4, 8, 32]),
                  min_lowbit_size=rnd.choice([4096, 1024]), quan_blocksize=rnd.choice([64, 128]), fused=True)
        if variant == "shampoo2":
            kw["inv_root_mode"] = rnd.choice([0, 1])
        Opt = rnd.choice([S.ShampooAdamW, S.ShampooSGD])
        if Opt is S.ShampooSGD:
            kw["momentum"] = 0.9
        steps, cut = 8, rnd.randint(1, 6)
        g = torch.Generator(device="cuda").manual_seed(seed)
        init = [0.1 * torch.randn(s, device="cuda", generator=g) for s in shapes]
        grads = [[0.05 * torch.randn(s, device="cuda", generator=g) for s in shapes] for _ in range(steps)]
        missing = {(st, pi) for st in range(steps) for pi in range(len(shapes)) if rnd.random() < 0.1}

        def step(params, opt, st):
            torch.manual_seed(777 + st)                    # the power iteration draws its start vectors from torch's generator
            for pi, p in enumerate(params):
                p.grad = None if (st, pi) in missing else grads[st][pi].clone()
            opt.step()

        params = [torch.nn.Parameter(t.clone()) for t in init]
        opt = Opt(params, **kw)
        for st in range(cut):
            step(params, opt, st)
        buf = io.BytesIO()
        torch.save({"opt": opt.state_dict(), "params": [p.detach().clone() for p in params]}, buf)
        buf.seek(0)
        for st in range(cut, steps):
            step(params, opt, st)
        saved = torch.load(buf, weights_only=True)
        again = [torch.nn.Parameter(t.clone()) for t in saved["params"]]
        opt2 = Opt(again, **kw)
        opt2.load_state_dict(saved["opt"])
        for st in range(cut, steps):
            step(again, opt2, st)
        torch.cuda.synchronize()
        for a, b in zip(params, again):
            assert bool(torch.isfinite(a).all()) and torch.equal(a.detach(), b.detach()), (variant, seed, shapes, kw, cut)
