"""Batched execution of the eigenbasis variant of low-bit Shampoo (the reference's shampoo2.py)
over all parameters at once.

Every statistic L is held as the reference's QTensorSVDFast holds it (qtensor/utils.py:124-236):
the quantized matrix Vt whose rows approximate eigenvectors, the smaller half of the Rayleigh
quotients, the rows they belong to and the largest quotient.  One statistics update is one step
of subspace iteration per matrix (shampoo2.py:185-200, utils.py:156-203):

    Vt <- 1.5 Vt - 0.5 Vt Vt^T Vt            (rect_t1 times, after dequantizing)
    L  <- b * Vt[keep]^T diag(S) Vt[keep] + (1 - b) * G G^T
    V  <- orthonormal basis of L Vt^T, columns in order (QR)
    quotients <- diag(V^T L V); keep the smaller half; store V^T quantized

Here all statistics of one order form a stack and every line above is one or two launches for
the whole stack: the products run on the matrix cores through qtensor.fused.gemm (symmetric
ones compute half and mirror), and the QR factorisation -- 20 ms per 1024 x 1024 matrix through
the vendor's Householder routine, 5 s per step for a ViT-B/32 -- is replaced by one sweep of
block Gram-Schmidt with reorthogonalisation per stack (panels of the column-scaled matrix left to
right; the products run on the matrix cores, the 64-column panels are orthonormalised by Cholesky
QR; batched launches of libqtensor_hip.so), checked afterwards and polished by a Cholesky QR round
where needed, which yields the same factor Q up to column signs.  Matrices that cannot be
finished this way are redone with torch.linalg.qr.
"""
import time

import torch

from optimizers.engine import LANES, ShampooBank, SideJob
from optimizers.matrix_functions import ComputePowerBatched
from qtensor import fused as X


cholesky_qr = X.cholesky_qr


class ShampooBank2(ShampooBank):
    # Two lanes for the large stacks, one for the small ones, one for the few matrices that are swept apart from
    # their stack (a process has four hardware queues; on the ViT-B/32 shapes fewer side streams cost a millisecond
    # or two per regular step, more gain nothing).
    DEFAULT_STREAMS = 4

    def __init__(self, params, name2qmap, code, *, rect_t1=1, rect_t2=4, inv_root_mode=0, **kwargs):
        self.rect_t1, self.rect_t2, self.inv_root_mode = rect_t1, rect_t2, inv_root_mode
        self.qr_fallbacks = 0                     # matrices that went through torch.linalg.qr so far
        self.qr_rounds = 0                        # Cholesky QR rounds so far, summed over the stacks
        self.qr_repairs = 0                       # matrices that went through the replacing sweep so far (low numerical rank)
        self.alongside = None                     # callable that the next add_statistics runs next to its factorisations
        self.low_rank = {}                        # order -> [most of the stack needed the replacing sweep, updates since the plain one was tried]
        self.low_rank_rows = {}                   # order -> {row: [updates between two looks at the plain sweep, updates until the next look]}
        super().__init__(params, name2qmap, code, **kwargs)
        # Statistics that cannot have full rank, whatever the gradients: the update of a block's statistic of order n is
        # b * (its kept half: rank n // 2) + (1 - b) * G G^T with G n x m, so its rank is at most n // 2 + m -- the order-768
        # statistic of a 768 x 256 block has a null space of 128 dimensions in every update.  order -> rows of its stack
        self.rank_deficient = self._rank_deficient_rows(self.groups)

    @staticmethod
    def _rank_deficient_rows(groups):
        rows = {}
        for g in groups:
            for side, (order, other) in enumerate(((g.bm, g.bn), (g.bn, g.bm))):
                if max(1, order // 2) + other < order:
                    first = g.slot[side][1]
                    rows.setdefault(order, []).extend(range(first, first + len(g)))
        return {order: sorted(r) for order, r in rows.items()}

    QUOTIENT_PART_BYTES = 128 << 20               # L Q for the Rayleigh quotients is formed this much at a time
    LOOK_AGAIN = 8                                # updates after which a stack of low numerical rank tries the plain sweep again
    STALL_SECONDS = 300.0                         # the host polls the device while the stacks are factored: not for ever

    def _replace_first(self, order):
        """Whether this update of the stack starts with the replacing sweep: its last update with the plain sweep
        needed the replacing one for more than a quarter of the matrices, fewer than LOOK_AGAIN updates ago."""
        state = self.low_rank.setdefault(order, [False, 0])
        if not state[0]:
            return False
        state[1] += 1
        if state[1] >= self.LOOK_AGAIN:
            state[1] = 0
            return False
        return True

    APART_AT_MOST = 32                            # so many known low-rank matrices of a stack are still orthonormalised on their own

    def _known_low_rank(self, order):
        """The matrices of this stack that are, for this update, taken to be of low numerical rank: those that cannot
        have full rank by the shape of their block (rank_deficient: the order-768 statistics of a 768 x 100 head and of
        the 768 x 256 blocks of a 768 x 2304 weight), and those whose recent updates ended in the replacing sweep.
        Up to APART_AT_MOST of them (and at most a quarter of the stack) are orthonormalised apart from their stack, as a
        small stack of their own that starts with the replacing sweep, on a stream next to the lanes, while the stack
        itself gets the plain sweep and leaves their places alone; with more of them the whole stack starts with the
        replacing sweep.  Every `period` updates a matrix of the second kind goes through the plain sweep with its stack
        again; the period doubles (8, 16, ... 256) each time that look ends in the replacing sweep once more."""
        known = set(self.rank_deficient.get(order, ()))
        for row, state in self.low_rank_rows.setdefault(order, {}).items():
            if state[1] > 0:
                state[1] -= 1
                known.add(row)
        return sorted(known)

    def _row_index(self, rows):
        """int64 device vector of a short list of row numbers, kept: a copy from the host in the middle of an update
        would make the host wait for the stream it is queued on."""
        cache = self.__dict__.setdefault("_row_index_cache", {})
        key = tuple(rows)
        if key not in cache:
            if len(cache) > 64:
                cache.clear()
            cache[key] = torch.tensor(list(rows), dtype=torch.int64, device=self.device)
        return cache[key]

    def _note_repairs(self, order, repaired):
        table = self.low_rank_rows.setdefault(order, {})
        for row in repaired:
            period = min(2 * table[row][0], 256) if row in table else 8
            table[row] = [period, period]

    def _init_statistics(self):
        """Basis = quantized identity, every kept quotient and the largest one = matrix_eps
        (reference: utils.py:134-153 with var = matrix_eps * I)."""
        self.basis, self.svalue, self.keep, self.max_eig = {}, {}, {}, {}
        for order, count in self.per_order.items():
            self.basis[order] = self._new_store(order, count, 1.0, False)
            half = max(1, order // 2)
            self.keep[order] = torch.arange(half, device=self.device).expand(count, half).contiguous()
            self.svalue[order] = torch.full((count, half), self.matrix_eps, device=self.device)
            self.max_eig[order] = torch.full((count,), self.matrix_eps, device=self.device)

    # ---- pieces of QTensorSVDFast, for a whole stack ---------------------------------------------
    def _pick(self, order, rows):
        """(basis, kept row indices, kept quotients, largest quotient) of the whole stack (rows None) or of a copy
        of the given rows of it."""
        if rows is None:
            return self.basis[order], self.keep[order], self.svalue[order], self.max_eig[order]
        return (self.basis[order].select(rows), self.keep[order].index_select(0, rows),
                self.svalue[order].index_select(0, rows), self.max_eig[order].index_select(0, rows))

    def _rectified_basis(self, order, rows=None):
        """Dequantized Vt after rect_t1 Bjorck steps (utils.py:194-198; a basis held in fp32 is used as it is)."""
        basis = self._pick(order, rows)[0]
        vt = X.load_stack(basis)
        if isinstance(basis, X.DenseStack):
            return vt
        for _ in range(self.rect_t1):
            vvt = X.gemm(vt, vt, trans_b=True, symmetric=True)
            vt = X.gemm(vvt, vt, addend=vt, alpha=-0.5, beta=1.5)
        return vt

    @staticmethod
    def _gather_rows(vt, keep):
        n = vt.shape[2]
        return torch.gather(vt, 1, keep.unsqueeze(2).expand(-1, -1, n))

    def _kept_rows(self, order, vt, rows=None):
        return self._gather_rows(vt, self._pick(order, rows)[1])

    def _statistic(self, order, vt, out=None, rows=None):
        """Vt[keep]^T diag(S) Vt[keep] (utils.py:200-203)."""
        _, keep, svalue, _ = self._pick(order, rows)
        kept = self._gather_rows(vt, keep)
        return X.gemm(kept * svalue.unsqueeze(2), kept, trans_a=True, symmetric=True, out=out)

    # ---- the operations of the reference's Preconditioner ----------------------------------------
    @torch.no_grad()
    def add_statistics(self, grads, only=None):
        """only: the indices of the parameters whose statistics are updated (default: all).  The stacks that hold
        a block of one of them are updated whole -- the other matrices of such a stack go through the same update
        without a gradient term -- and only the rows of the chosen parameters are written back."""
        only = self._only(only, len(self.params))
        self._check(grads, only)
        w1 = self.stat_decay
        w2 = 1.0 if w1 == 1.0 else 1.0 - w1
        orders = [o for o in sorted(self.per_order, key=lambda o: -o ** 3 * self.per_order[o]) if self._touched(o, only)]
        if not orders:
            return
        # buffers that cross the phases below belong to the current stream
        stat = {o: torch.empty(self.per_order[o], o, o, device=self.device) for o in orders}
        basis = {}
        for g in self.groups:
            self._grad_list(g, grads)

        solver, redone, tick, begun = {}, {}, {}, {}
        # (a stack starts with the replacing sweep when most of it needed that sweep lately, or when it holds many
        # matrices that did; a few such matrices are orthonormalised apart from it)
        direct, apart = {}, {}
        for o in orders:
            mostly, known = self._replace_first(o), self._known_low_rank(o)
            direct[o] = mostly or len(known) > self.APART_AT_MOST or 4 * len(known) > self.per_order[o]
            apart[o] = [] if direct[o] else known
        apart_y, apart_event, apart_q, apart_back = {}, {}, {}, {}

        def rebuild(order):
            def run():
                basis[order] = self._rectified_basis(order)
                self._statistic(order, basis[order], out=stat[order])
            return run

        def accumulate(g, side):
            def run():
                order, first = g.slot[side]
                seg = stat[order][first:first + len(g)]
                G = self._grad_list(g, grads)
                X.gemm(G, G, trans_a=side == 1, trans_b=side == 0, addend=seg, alpha=w2, beta=w1, out=seg, symmetric=True,
                       skip=self._skip(g, only))
            return run

        def project(order):
            def run():
                # L Vt^T.  The product is given up to the solver (scaled in place, it becomes Q) and the rectified basis
                # is let go right here: from now on a stack holds its statistic and Q.  The few matrices whose columns
                # are needed once more (low numerical rank: swept again from the original columns) are made anew.
                def remake(ids):
                    return X.gemm(stat[order].index_select(0, ids), self._rectified_basis(order, ids), trans_b=True)

                product = X.gemm(stat[order], basis[order], trans_b=True)
                begun[order] = torch.cuda.Event()
                begun[order].record(torch.cuda.current_stream(self.device))
                if apart[order]:
                    # the columns of the matrices that go their own way, before the product is scaled in place
                    apart_y[order] = product.index_select(0, self._row_index(apart[order]))
                    apart_event[order] = torch.cuda.Event()
                    apart_event[order].record(torch.cuda.current_stream(self.device))
                basis[order] = None
                solver[order] = X.CholeskyQR(product, replace_first=direct[order], remake=remake, leave=apart[order])
                del product
                # (the event that tells the host this stack's sweep is through goes right behind it: streams share
                # hardware queues, and behind the launches of another stack's sweep it would wait for those as well)
                tick[order] = torch.cuda.Event()
                tick[order].record(torch.cuda.current_stream(self.device))
            return run

        def iterate(order):
            def run():
                L = stat[order]
                Q, redone[order] = solver[order].result()
                if apart[order]:                       # the matrices that went apart come back into their places
                    torch.cuda.current_stream(self.device).wait_event(apart_back[order])
                    own = apart_q.pop(order)
                    Q.index_copy_(0, self._row_index(apart[order]), own)
                    own.record_stream(torch.cuda.current_stream(self.device))
                # Rayleigh quotients diag(Q^T L Q), the product L Q a few dozen matrices at a time
                quotients = torch.empty(Q.shape[0], Q.shape[1], device=self.device)
                per = max(1, self.QUOTIENT_PART_BYTES // (4 * order * order))
                for first in range(0, Q.shape[0], per):
                    q = Q[first:first + per]
                    lq = X.gemm(L[first:first + per], q)
                    quotients[first:first + per] = X.column_dots(q, lq) if order % 64 == 0 else (q * lq).sum(dim=1)
                del lq
                ascending, where = torch.sort(quotients, dim=1)
                half = self.keep[order].shape[1]
                rows = self._rows(order, only)
                if rows is None:
                    self.keep[order] = where[:, :half].contiguous()
                    self.svalue[order] = ascending[:, :half].contiguous()
                    self.max_eig[order] = quotients.amax(dim=1)
                    X.store_stack(Q, self.basis[order], transposed=True)               # rows of the stored matrix = columns of Q
                else:                                                                  # only the chosen parameters' rows change
                    self.keep[order].index_copy_(0, rows, where[:, :half].index_select(0, rows))
                    self.svalue[order].index_copy_(0, rows, ascending[:, :half].index_select(0, rows))
                    self.max_eig[order].index_copy_(0, rows, quotients.amax(dim=1).index_select(0, rows))
                    chosen = Q.index_select(0, rows)
                    self.basis[order].put(rows, X.store_stack(chosen, self.basis[order].select(rows), transposed=True))
            return run

        gradient_terms = {o: [] for o in orders}              # order -> the products G G^T / G^T G that go into its stack
        for g in self.groups:
            if only is None or any(pi in only for pi in g.param_index):
                for side in (0, 1):
                    gradient_terms[g.slot[side][0]].append(accumulate(g, side))
        # The Cholesky QR of every order advances on its own stream; the host waits once per round.
        # (_fan_out gives job i the stream i % streams, so an order keeps its stream from call to call.)
        # Two lanes for the sweeps and what follows them, a third for stacks of a matrix or two: a process has four
        # hardware queues, the current stream takes one, and streams beyond that share a queue in the order of their
        # launches -- a third large stack on a stream of its own ran behind the second anyway, and held up what the
        # second had to do after its sweep.  The stacks are dealt out by cost, the cheap ones of a lane first.
        cost = {o: o ** 3 * self.per_order[o] for o in orders}
        small = [o for o in orders if cost[o] * 50 < max(cost.values())]          # a matrix or two of a small order: a chain of tiny launches
        big = [o for o in orders if o not in small]
        lanes = [[] for _ in range(min(LANES, len(big)))]
        for o in big:                                                      # (most expensive first)
            min(lanes, key=lambda lane: sum(cost[x] for x in lane)).append(o)
        lanes = [sorted(lane, key=lambda x: cost[x]) for lane in lanes]
        if small:                                                          # (they get a lane of their own: nothing big waits behind them)
            lanes.append(sorted(small, key=lambda x: cost[x]))
        slot = {o: i for i, lane in enumerate(lanes) for o in lane}
        # (index tensors of the matrices that go apart, made before anything is queued)
        for o in orders:
            if apart[o]:
                self._row_index(apart[o])
        # (a stream of their own, next to the lanes: behind their long chain of small launches the host would wait
        # with every test of a small stack)
        apart_lane = len(lanes)
        keys = list(orders) + [(o, "apart") for o in orders if apart[o]]
        for o in orders:
            if apart[o]:
                slot[(o, "apart")] = apart_lane

        def sweep_apart(order):
            def run():
                # the known low-rank matrices of the stack as a stack of their own, replacing sweep first
                current = torch.cuda.current_stream(self.device)
                current.wait_event(apart_event[order])
                y = apart_y.pop(order)
                y.record_stream(current)                                   # (made on the stack's lane, used up on this one)
                ids = self._row_index(apart[order])

                def remake(which):
                    rows = ids.index_select(0, which)
                    return X.gemm(stat[order].index_select(0, rows), self._rectified_basis(order, rows), trans_b=True)

                key = (order, "apart")
                solver[key] = X.CholeskyQR(y, replace_first=True, remake=remake)
                tick[key] = torch.cuda.Event()
                tick[key].record(current)
            return run

        def chain(lane):
            def run():
                # a stack is rebuilt, takes its gradient terms, is multiplied out and swept on its lane, one stack of
                # the lane after the other; the lanes start together and nothing waits for another lane on the way
                # (the second lane held back until the first one's large products are through, so that they fill the
                # device next to the other lane's sweep and not next to each other, is a millisecond slower per step)
                for o in lane:
                    rebuild(o)()
                    for job in gradient_terms[o]:
                        job()
                    project(o)()
            return run

        jobs = [chain(lane) for lane in lanes]
        if any(apart.values()):
            own = [sweep_apart(o) for o in orders if apart[o]]
            jobs.append(lambda: [job() for job in own])
        self._fan_out(jobs, join=False)
        # Work of the caller that does not depend on the statistics (bank.alongside, consumed here) fills the device
        # next to the sweeps -- chains of launches that leave most of it idle -- and not next to the large products
        # before them: it goes to the current stream, which has nothing else to do until all stacks are through (it
        # waits for them at the very end), behind the point where the first lane's sweep begins, and is queued by a
        # thread of its own.  (A further stream would share a hardware queue with one of the lanes and run behind
        # that lane's sweep, and that lane's next step behind it.)
        beside, self.alongside = self.alongside, None
        if beside is not None:
            current = torch.cuda.current_stream(self.device)
            current.wait_event(begun[lanes[0][0]])
            beside = SideJob(self.device, current, beside)
        # Every stack goes on alone from here, on the stream that holds its sweep: the test after the sweep (the host
        # reads the sweep's flags, then the deviations of the flagged matrices), a polishing round where needed, and
        # as soon as it is finished its Rayleigh quotients and re-encoding -- none of it waits for the sweep of another
        # stack (the current stream, which waits for all of them, is left out of it).  The host takes the stacks in the
        # order in which their streams get there: it polls an event per stack.
        def cost_of(key):
            return key ** 3 * self.per_order[key] if not isinstance(key, tuple) else key[0] ** 3 * len(apart[key[0]])

        unfinished = sorted(keys, key=cost_of)
        on_side = bool(self.streams)

        def tick_of(key):
            event = torch.cuda.Event()
            event.record(self.streams[slot[key] % len(self.streams)] if on_side else torch.cuda.current_stream(self.device))
            return event

        tested = {k: False for k in keys}              # the test of the current iterate is queued, its outcome not read yet

        def look_at(key):
            # one step of the stack's state machine; every read of the host in it finds its data there already,
            # because the step before it ended with the event that is now through
            def run():
                s = solver[key]
                if not tested[key]:
                    s.check()
                    tested[key] = not s.finished
                else:
                    tested[key] = False
                    if not s.poll():
                        s.advance()
            return run

        def hand_back(order):
            def run():
                # (result() on the stream the solver lived on; the stack's lane waits for the event)
                apart_q[order], redone[(order, "apart")] = solver[(order, "apart")].result()
                apart_back[order] = torch.cuda.Event()
                apart_back[order].record(torch.cuda.current_stream(self.device))
            return run

        waiting_since = time.monotonic()
        done = set()
        try:
            while unfinished:
                ready = [k for k in unfinished if tick[k].query()]
                if not ready:
                    if time.monotonic() - waiting_since > self.STALL_SECONDS:
                        raise RuntimeError(f"the statistics update of the orders {unfinished} made no progress on the device "
                                           f"for {self.STALL_SECONDS} s")
                    time.sleep(2e-5)
                    continue
                waiting_since = time.monotonic()
                for k in sorted(ready, key=lambda x: -cost_of(x)):
                    self._run_on(slot[k], look_at(k), after_current=False, join=False)
                    if not solver[k].finished:
                        tick[k] = tick_of(k)
                        continue
                    unfinished.remove(k)
                    done.add(k)
                    order = k[0] if isinstance(k, tuple) else k
                    if isinstance(k, tuple):
                        self._run_on(slot[k], hand_back(order), after_current=False, join=False)
                    # a stack goes on when it and the matrices that went apart from it are both through
                    if order in done and (not apart[order] or (order, "apart") in done):
                        self._run_on(slot[order], iterate(order), after_current=False, join=False)
        finally:
            if beside is not None:
                beside.join()
            self._join()
        self.qr_fallbacks += sum(redone.values())
        self.qr_rounds += sum(solver[k].rounds for k in keys)
        self.qr_repairs += sum(solver[k].repairs for k in keys)
        for o in orders:
            if not direct[o]:
                self.low_rank[o][0] = solver[o].repairs * 4 > self.per_order[o]
                self._note_repairs(o, solver[o].repaired_ids)

    @torch.no_grad()
    def compute_preconditioners(self, v0=None, only=None):
        """inv_root_mode 0: inverse 4th root from the stored eigenpairs (functional.py:749-762 through
        utils.py:205-227); 1: coupled Newton on the rebuilt statistic.  v0, only as in ShampooBank."""
        only = self._only(only, len(self.params))
        orders = [o for o in sorted(self.per_order, key=lambda o: -o ** 3 * self.per_order[o]) if self._touched(o, only)]
        starts = {}
        if self.inv_root_mode != 0:
            starts = {o: (torch.rand(self.per_order[o], o, device=self.device) * 2 - 1) if v0 is None else v0[o]
                      for o in self.per_order}

        def job(order):
            def run():
                rows = self._rows(order, only)
                for part in self._newton_parts(order, rows):
                    # (a part of the whole stack is gathered like a chosen set of rows: one copy of its 4-bit basis)
                    index = torch.arange(part[0], part[0] + part[1], device=self.device) if rows is None else part
                    whole = rows is None and part[1] == self.per_order[order]
                    basis, keep, svalue, max_eig = self._pick(order, None if whole else index)
                    if self.inv_root_mode == 0:
                        kept = self._gather_rows(X.load_stack(basis), keep)
                        if not isinstance(basis, X.DenseStack):          # (a basis held in fp32 is not rectified: utils.py:205-227)
                            for _ in range(self.rect_t2):
                                vvt = X.gemm(kept, kept, trans_b=True, symmetric=True)
                                kept = X.gemm(vvt, kept, addend=kept, alpha=-0.5, beta=1.5)
                        ridge = self.matrix_eps * max_eig
                        weights = 1 / (svalue + ridge.unsqueeze(1)).pow(1 / 4)
                        roots = X.gemm(kept * weights.unsqueeze(2), kept, trans_a=True, symmetric=True)
                    else:
                        L = self._statistic(order, self._rectified_basis(order, None if whole else index), rows=None if whole else index)
                        start = starts[order] if whole else starts[order].index_select(0, index)
                        # L is symmetric up to the rounding inside its diagonal tiles: half products are fine
                        roots = ComputePowerBatched(L, 4, ridge_epsilon=self.matrix_eps, v0=start, symmetric=True)
                    if rows is None:
                        X.store_stack(roots, self.precs[order].rows(part[0], part[1]))
                    else:
                        self.precs[order].put(index, X.store_stack(roots, self.precs[order].select(index)))
            return run

        self._fan_out([job(o) for o in orders], inline=not self.NEWTON_SIDE_BY_SIDE)
        for pi in range(len(self.params)):
            if only is None or pi in only:
                self.active[pi] = True

    # ---- checkpoints -----------------------------------------------------------------------------
    def _tensors(self):
        out = {}
        for order in self.per_order:
            self._store_tensors(f"basis.{order}", self.basis[order], out)
            out[f"basis.{order}.svalue"], out[f"basis.{order}.keep"] = self.svalue[order], self.keep[order]
            out[f"basis.{order}.max_eigenvalue"] = self.max_eig[order]
            self._store_tensors(f"precs.{order}", self.precs[order], out)
        return out

    def state_dict(self):
        # (which sweep a stack starts with is part of the state: a resumed run then takes the same sweeps and ends in
        # the same codes as an uninterrupted one)
        low_rank = torch.tensor([[o, int(state[0]), int(state[1])] for o, state in sorted(self.low_rank.items())],
                                dtype=torch.int64).reshape(-1, 3)
        rows = torch.tensor([[o, row, state[0], state[1]] for o, table in sorted(self.low_rank_rows.items())
                             for row, state in sorted(table.items())], dtype=torch.int64).reshape(-1, 4)
        return {**super().state_dict(), "low_rank": low_rank, "low_rank_rows": rows}

    def load_state_dict(self, sd):
        super().load_state_dict(sd)
        if "low_rank" in sd:
            self.low_rank = {int(o): [bool(flag), int(count)] for o, flag, count in sd["low_rank"].tolist()}
        if "low_rank_rows" in sd:
            self.low_rank_rows = {}
            for o, row, period, left in sd["low_rank_rows"].tolist():
                self.low_rank_rows.setdefault(int(o), {})[int(row)] = [int(period), int(left)]
