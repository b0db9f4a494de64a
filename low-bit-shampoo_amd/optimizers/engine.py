"""Batched execution of the "naive" low-bit Shampoo preconditioner over all parameters at once.

The reference walks parameters, blocks and sides in Python and issues a handful of small
kernels for each of them (optimizers/shampoo1.py:148-241, called per parameter from
:371-427).  A ViT-B/32 has 124 blocks and 248 statistics of only four distinct orders, so the
same arithmetic is done here with one launch per group of equally shaped blocks:

  statistics   L <- b L + (1-b) G G^T : one fused product per (block shape, side) that reads the
               quantized L inside its epilogue and writes the result back re-encoded (blocksize 64;
               other blocksizes: fp32 result, then one stack quantize)
  inverse root one stack dequantize, one batched sync-free Newton run, one stack quantize per order
  P_L G P_R    two fused products per block shape, the quantized factors expanded on the fly

The quantized state of all blocks of one order lives in one stacked allocation
(codes [B, n*n/2], maxima [B, n*ceil(n/bs)], diagonals [B, n]); entry b is bit-for-bit what
quantize_blockwise_diagreal writes for that matrix.  An order that the blocksize does not divide
(the 100 of a 768 x 100 head) is stored in the same format but cannot be read by the products
directly: its stack is dequantized, updated by dense products and quantized again.  An order
with fewer than min_lowbit_size elements, and every order with prec_bits = 32, is a plain fp32
stack, as the reference's holders keep such matrices (qtensor/utils.py:11-17).

Every operation takes an optional set of parameters to work on (`only`): the reference counts
steps per parameter and skips a parameter without a gradient (optimizers/shampoo1.py:371-377),
so the parameters of a bank may be due for different things at one call.
"""
import threading
from collections import defaultdict

import torch

from optimizers.matrix_functions import ComputePowerBatched
from optimizers.shampoo_common import BlockPartitioner
from qtensor import fused as X


class _Group:
    """All blocks of one (rows, cols, leading dimension) shape."""

    def __init__(self, bm, bn, ld):
        self.bm, self.bn, self.ld = bm, bn, ld
        self.param_index, self.offset = [], []       # which parameter, element offset of the block
        self.slot = [None, None]                     # (order, first row in that order's stack) per side
        self.grad_key, self.grad_ptrs, self.out_ptrs = None, None, None

    def __len__(self):
        return len(self.param_index)


_SHARED_STREAMS = {}
LANES = 2                                            # chains of launches the eigenbasis bank runs side by side


def shared_stream(device, slot):
    """Side stream number `slot` of the device, the same object for every bank and optimizer of the process (a
    second optimizer with streams of its own would double the chains that compete for the device's few hardware
    queues).  A dozen plain streams of default priority per device, made together on first use."""
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _SHARED_STREAMS:
        with torch.cuda.device(index):
            _SHARED_STREAMS[index] = [torch.cuda.Stream(device=index) for _ in range(12)]
    pool = _SHARED_STREAMS[index]
    return pool[slot % len(pool)]


class SideJob:
    """Runs fn() on a thread of its own with `stream` as that thread's current stream, ordered after what the
    caller's current stream holds now (`stream` may be that very stream: then only the queueing is done
    elsewhere); join() makes the caller's stream wait for it and passes an exception on."""

    def __init__(self, device, stream, fn):
        self.main, self.side, self.error = torch.cuda.current_stream(device), stream, None
        self.side.wait_stream(self.main)

        def run():
            try:
                torch.cuda.set_device(device)
                with torch.no_grad(), torch.cuda.stream(self.side):       # grad mode and current stream are per thread
                    fn()
            except BaseException as exc:                                   # noqa: BLE001 -- handed to join()
                self.error = exc

        self.thread = threading.Thread(target=run, name="shampoo-side-job")
        self.thread.start()

    def join(self):
        self.thread.join()
        self.main.wait_stream(self.side)
        if self.error is not None:
            raise self.error


class ShampooBank:
    DEFAULT_STREAMS = 3          # side streams for independent groups (0: everything on the current stream)

    def __init__(self, params, name2qmap, code, stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1200,
                 prec_bits=4, min_lowbit_size=4096, quan_blocksize=64, streams=None):
        self.stat_decay, self.matrix_eps = stat_decay, matrix_eps
        self.bits, self.blocksize, self.min_lowbit_size = prec_bits, quan_blocksize, min_lowbit_size
        self.params = list(params)
        self.device = self.params[0].device
        if prec_bits in (4, 8):
            self.code = name2qmap[code].to(self.device)
            name2qmap[code] = self.code
        else:
            self.code = None
        self.shapes = []                              # matrix view (m, n) of every parameter
        groups = {}
        for pi, p in enumerate(self.params):
            m, n = self.matrix_shape(p)
            self.shapes.append((m, n))
            part = BlockPartitioner(torch.empty(m, n, device="meta"), prec_maxorder)
            rows = self._pieces(m, prec_maxorder)
            cols = self._pieces(n, prec_maxorder)
            assert len(part.shapes_for_preconditioners()) == 2 * len(rows) * len(cols)
            r0 = 0
            for bm in rows:
                c0 = 0
                for bn in cols:
                    g = groups.setdefault((bm, bn, n), _Group(bm, bn, n))
                    g.param_index.append(pi)
                    g.offset.append(r0 * n + c0)
                    c0 += bn
                r0 += bm
        self.groups = list(groups.values())
        per_order = defaultdict(int)
        for g in self.groups:
            for side, order in enumerate((g.bm, g.bn)):
                g.slot[side] = (order, per_order[order])
                per_order[order] += len(g)
        self.per_order = dict(per_order)
        too_many = {o: c for o, c in self.per_order.items() if c > 65535}
        if too_many:
            raise ValueError(f"the batched engine takes at most 65535 blocks per order in one launch, got {too_many}; "
                             "use a larger prec_maxorder or the per-parameter path (fused=False)")
        self.precs = {order: self._new_store(order, count, 1.0, True) for order, count in per_order.items()}
        self._init_statistics()
        self.active = [False] * len(self.params)      # per parameter: its inverse roots have been computed at least once
        self._rows_cache, self._skip_cache = {}, {}
        # Independent groups run on a few side streams so that the tail of one launch overlaps the
        # head of the next; biggest first.
        self.groups.sort(key=lambda g: -len(g) * g.bm * g.bn * (g.bm + g.bn))
        streams = self.DEFAULT_STREAMS if streams is None else streams
        self.streams = [shared_stream(self.device, i) for i in range(min(streams, len(self.groups), 8))]

    # ---- storage ---------------------------------------------------------------------------------
    def lowbit(self, order):
        """Whether the matrices of this order are stored quantized (the rule of the reference's holders)."""
        return self.bits in (4, 8) and order * order >= self.min_lowbit_size

    def _new_store(self, order, count, scale, diagreal):
        """A stack of `count` matrices scale * I of this order in the bank's storage format."""
        eye = torch.zeros(count, order, order, device=self.device)
        eye.diagonal(dim1=1, dim2=2).fill_(scale)
        if not self.lowbit(order):
            return X.DenseStack(eye)
        return X.quantize_stack(eye, X.empty_quantized(count, order, self.blocksize, self.bits, self.code, diagreal))

    def _init_statistics(self):
        """Statistics start as matrix_eps * I, stored quantized with an exact diagonal."""
        self.stats = {order: self._new_store(order, count, self.matrix_eps, True) for order, count in self.per_order.items()}

    def _landing(self, g, side):
        """fp32 landing area of an updated statistic stack (only for blocksizes the requantizing product does not take)."""
        if getattr(g, "scratch", None) is None:
            g.scratch = [None, None]
        if g.scratch[side] is None:
            order = (g.bm, g.bn)[side]
            g.scratch[side] = torch.empty(len(g), order, order, device=self.device)
        return g.scratch[side]

    def _fan_out(self, jobs, inline=False, join=True):
        """Run the callables round-robin on the side streams, after everything already queued on the
        current stream; the current stream then waits for all of them (join=False: the caller does that
        later, with _join).  inline: one after the other on the current stream (for a caller that is itself
        a side job next to another fan-out)."""
        if inline or not self.streams:
            for job in jobs:
                job()
            return
        main = torch.cuda.current_stream(self.device)
        start = torch.cuda.Event()
        start.record(main)
        for i, job in enumerate(jobs):
            side = self.streams[i % len(self.streams)]
            if i < len(self.streams):
                side.wait_event(start)
            with torch.cuda.stream(side):
                job()
        if join:
            self._join(len(jobs))

    def _join(self, count=None):
        """The current stream waits for what the first `count` side streams (default: all) hold now."""
        main = torch.cuda.current_stream(self.device)
        for side in self.streams[:count]:
            main.wait_stream(side)

    def _run_on(self, slot, job, after_current=True, join=True):
        """Run one callable on side stream `slot` (the stream _fan_out gives job number `slot`), after what the
        current stream holds; the current stream then waits for it (join=False: the caller does that later, with
        _join).  after_current=False: only after what that side stream holds itself -- for a job that goes on with
        the work of an earlier job on the same stream, while the current stream has since moved on."""
        if not self.streams:
            job()
            return
        main = torch.cuda.current_stream(self.device)
        side = self.streams[slot % len(self.streams)]
        if after_current:
            side.wait_stream(main)
        with torch.cuda.stream(side):
            job()
        if join:
            main.wait_stream(side)

    # ---- eligibility -----------------------------------------------------------------------------
    @staticmethod
    def matrix_shape(p):
        dims = [d for d in p.shape if d != 1]
        if len(dims) <= 1:
            return None
        first = dims[0]
        return first, p.numel() // first

    @staticmethod
    def _pieces(extent, block):
        if block > 0 and extent > block:
            cuts = (extent - 1) // block
            return [block] * cuts + [extent - cuts * block]
        return [extent]

    @classmethod
    def accepts(cls, p, prec_maxorder, prec_bits, min_lowbit_size, quan_blocksize):
        """A parameter can live in the bank when it is an fp32 GPU tensor with a matrix view (two or more
        dimensions that are not 1) and the bit width is one the bank stores (4, 8: quantized; 32: fp32)."""
        if not p.is_cuda or p.dtype != torch.float32 or prec_bits not in (4, 8, 32):
            return False
        return cls.matrix_shape(p) is not None

    # ---- per-step plumbing -----------------------------------------------------------------------
    def _segment(self, table, g, side):
        order, first = g.slot[side]
        return table[order].rows(first, len(g))

    def _grad_list(self, g, grads):
        # (a parameter that is left out of this call has no gradient: its own storage stands in, never read)
        key = tuple((self.params[pi] if grads[pi] is None else grads[pi]).data_ptr() for pi in g.param_index)
        if key != g.grad_key:
            g.grad_ptrs = torch.tensor([base + 4 * off for base, off in zip(key, g.offset)], dtype=torch.int64,
                                       device=self.device)
            g.grad_key = key
        return X.PtrList(g.grad_ptrs, (len(g), g.bm, g.bn), ld=g.ld)

    def _out_list(self, g):
        if g.out_ptrs is None:
            g.out_ptrs = torch.tensor([self.outputs[pi].data_ptr() + 4 * off for pi, off in zip(g.param_index, g.offset)],
                                      dtype=torch.int64, device=self.device)
        return X.PtrList(g.out_ptrs, (len(g), g.bm, g.bn), ld=g.ld)

    def _check(self, grads, only=None):
        if len(grads) != len(self.params):
            raise ValueError("one gradient per parameter, in the order given at construction")
        for pi, (grad, (m, n)) in enumerate(zip(grads, self.shapes)):
            if only is not None and pi not in only:
                continue
            if grad is None:
                raise ValueError("a parameter that takes part in this call needs a gradient")
            if grad.numel() != m * n or not grad.is_contiguous() or grad.dtype != torch.float32 or not grad.is_cuda:
                raise ValueError("gradients must be contiguous fp32 GPU tensors of the parameters' shapes")

    @staticmethod
    def _only(only, count):
        """None when every parameter takes part, else the frozenset of those that do."""
        if only is None:
            return None
        only = frozenset(only)
        return None if len(only) == count and all(0 <= i < count for i in only) else only

    def _skip(self, g, only):
        """int32 [len(g)] with 1 for the blocks of parameters that are left out (None: none is)."""
        if only is None:
            return None
        key = (id(g), only)
        if key not in self._skip_cache:
            if len(self._skip_cache) > 64:
                self._skip_cache.clear()
            flags = [0 if pi in only else 1 for pi in g.param_index]
            self._skip_cache[key] = torch.tensor(flags, dtype=torch.int32, device=self.device) if any(flags) else None
        return self._skip_cache[key]

    def _rows(self, order, only):
        """int64 vector of the rows of this order's stacks that belong to the parameters in `only` (None: all rows)."""
        if only is None:
            return None
        key = (order, only)
        if key not in self._rows_cache:
            if len(self._rows_cache) > 64:
                self._rows_cache.clear()
            rows = [first + i for g in self.groups for (o, first) in g.slot if o == order
                    for i, pi in enumerate(g.param_index) if pi in only]
            full = len(rows) == self.per_order[order]
            self._rows_cache[key] = None if full else torch.tensor(sorted(rows), dtype=torch.int64, device=self.device)
        return self._rows_cache[key]

    def _touched(self, order, only):
        """Whether any row of this order belongs to a parameter in `only`."""
        rows = self._rows(order, only)
        return rows is None or rows.numel() > 0

    def prepare(self, grads, only=None):
        """Checks the gradients and writes the device tables of their block addresses, so that operations
        started afterwards from several threads only read them."""
        only = self._only(only, len(self.params))
        self._check(grads, only)
        for g in self.groups:
            self._grad_list(g, grads)

    # The coupled Newton iteration holds ten fp32 stacks of what it works on (two copies each of the root, the
    # iterate and the iteration matrix, two powers, the input, the result): a stack goes through it in parts of
    # at most this many bytes, one after the other, so that the iteration of a whole model takes ten times this
    # much scratch and not ten times its largest stack (ViT-B/32: 70.1 ms per step with inverse roots and 1.8 GiB of
    # scratch, against 68.8 ms and 4.2 GiB with whole stacks).  (A part still is dozens of matrices: every product launch
    # has thousands of tiles; the bits of a matrix's root do not depend on how its stack is cut.)
    NEWTON_PART_BYTES = 160 << 20
    NEWTON_SIDE_BY_SIDE = True                   # the orders' iterations run side by side on the side streams (False: one after the other)

    def _newton_parts(self, order, rows):
        """The stack of this order in parts for the Newton iteration: (first, count) ranges of the whole stack
        (rows None), else pieces of the int64 vector of rows."""
        per = max(1, self.NEWTON_PART_BYTES // (4 * order * order))
        if rows is None:
            count = self.per_order[order]
            return [(first, min(per, count - first)) for first in range(0, count, per)]
        return list(rows.split(per))

    # ---- the three operations of the reference's Preconditioner, for all parameters at once ------
    @torch.no_grad()
    def add_statistics(self, grads, only=None):
        """only: the indices of the parameters whose statistics are updated (default: all)."""
        only = self._only(only, len(self.params))
        self._check(grads, only)
        w1 = self.stat_decay
        w2 = 1.0 if w1 == 1.0 else 1.0 - w1

        def job(g, side):
            def run():
                G = self._grad_list(g, grads)
                seg = self._segment(self.stats, g, side)
                skip = self._skip(g, only)
                kw = dict(trans_a=side == 1, trans_b=side == 0, alpha=w2, beta=w1, symmetric=True)
                if seg.flat and self.blocksize == 64:
                    # dequantize, update and requantize in one launch: the fp32 statistic never reaches memory
                    X.gemm(G, G, addend=seg, requantize=True, skip=skip, **kw)
                    return
                if skip is None:
                    if seg.flat:
                        out = self._landing(g, side)
                        X.gemm(G, G, addend=seg, out=out, **kw)
                    else:                               # dense products on the dequantized (or fp32) stack
                        out = X.load_stack(seg)
                        X.gemm(G, G, addend=out, out=out, **kw)
                    X.store_stack(out, seg)
                    return
                # some blocks are left out: the others are gathered, updated and put back
                take = torch.nonzero(skip == 0).squeeze(1)
                sub = seg.select(take)
                dense = X.load_stack(sub)
                X.gemm(X.PtrList(G.ptrs.index_select(0, take), (take.numel(), g.bm, g.bn), ld=g.ld),
                       X.PtrList(G.ptrs.index_select(0, take), (take.numel(), g.bm, g.bn), ld=g.ld),
                       addend=dense, out=dense, **kw)
                seg.put(take, X.store_stack(dense, sub))
            return run

        for g in self.groups:           # address tables are written on the current stream, before the fan-out
            self._grad_list(g, grads)
        self._fan_out([job(g, side) for g in self.groups for side in (0, 1)
                       if only is None or any(pi in only for pi in g.param_index)])

    @torch.no_grad()
    def compute_preconditioners(self, v0=None, only=None):
        """v0: optional dict order -> [count, order] start vectors of the power iteration.
        only: the indices of the parameters whose inverse roots are computed (default: all)."""
        only = self._only(only, len(self.params))

        def job(order):
            def run():
                rows = self._rows(order, only)
                for part in self._newton_parts(order, rows):
                    if rows is None:
                        first, count = part
                        stat, target = self.stats[order].rows(first, count), self.precs[order].rows(first, count)
                        start = starts[order][first:first + count]
                    else:
                        stat, target = self.stats[order].select(part), self.precs[order].select(part)
                        start = starts[order].index_select(0, part)
                    # (an fp32 statistic is handed over as it is and keeps the ridge that the iteration adds in
                    # place, as in the reference: optimizers/shampoo1.py:198)
                    dense = X.load_stack(stat)
                    roots = ComputePowerBatched(dense, 4, ridge_epsilon=self.matrix_eps, v0=start)
                    X.store_stack(roots, target)
                    if rows is not None:
                        if isinstance(stat, X.DenseStack):
                            self.stats[order].put(part, stat)
                        self.precs[order].put(part, target)
            return run

        # start vectors come from the global generator in a fixed order, whatever the streams do
        starts = {order: (torch.rand(stat.batch, order, device=self.device) * 2 - 1) if v0 is None else v0[order]
                  for order, stat in self.stats.items()}
        orders = [o for o in sorted(self.stats, key=lambda o: -o ** 3 * self.stats[o].batch) if self._touched(o, only)]
        self._fan_out([job(order) for order in orders], inline=not self.NEWTON_SIDE_BY_SIDE)
        for pi in range(len(self.params)):
            if only is None or pi in only:
                self.active[pi] = True

    def _ensure_outputs(self):
        if getattr(self, "outputs", None) is None:
            self.outputs = [torch.empty(m, n, device=self.device) for m, n in self.shapes]
            for g in self.groups:
                g.out_ptrs = None

    @torch.no_grad()
    def preconditioned_grads(self, grads, inline=False, only=None):
        """List of P_L G P_R per parameter (buffers owned by the bank, overwritten by the next call; None for a
        parameter that `only` leaves out).  inline: every launch on the current stream."""
        only = self._only(only, len(self.params))
        self._check(grads, only)
        self._ensure_outputs()

        def job(g):
            def run():
                skip = self._skip(g, only)
                left, right = self._segment(self.precs, g, 0), self._segment(self.precs, g, 1)
                left = left if left.flat else X.load_stack(left)         # read inside the product, or dequantized first
                right = right if right.flat else X.load_stack(right)
                half = torch.empty(len(g), g.bm, g.bn, device=self.device)
                X.gemm(left, self._grad_list(g, grads), out=half, skip=skip)
                X.gemm(half, right, out=self._out_list(g), skip=skip)
            return run

        for g in self.groups:
            self._grad_list(g, grads)
            self._out_list(g)
        self._fan_out([job(g) for g in self.groups if only is None or any(pi in only for pi in g.param_index)], inline=inline)
        return [out.view(p.shape) if only is None or pi in only else None
                for pi, (out, p) in enumerate(zip(self.outputs, self.params))]

    def is_active(self):
        return all(self.active)

    # ---- inspection (tests, checkpoints) ---------------------------------------------------------
    def block_table(self):
        """[(parameter index, block index within the parameter (row-major), side, order, row in that
        order's stack)] -- where every statistic / preconditioner of the per-parameter layout lives."""
        per_param = defaultdict(list)
        for g in self.groups:
            for i, (pi, off) in enumerate(zip(g.param_index, g.offset)):
                per_param[pi].append((off, g, i))
        rows = []
        for pi in sorted(per_param):
            n = self.shapes[pi][1]
            items = sorted(per_param[pi], key=lambda t: (t[0] // n, t[0] % n))
            for j, (_, g, i) in enumerate(items):
                for side in (0, 1):
                    order, first = g.slot[side]
                    rows.append((pi, j, side, order, first + i))
        return rows

    @staticmethod
    def _store_tensors(prefix, store, out):
        if isinstance(store, X.DenseStack):
            out[prefix + ".dense"] = store.data
            return
        out[prefix + ".codes"], out[prefix + ".absmax"] = store.codes, store.absmax
        if store.diag is not None:
            out[prefix + ".diag"] = store.diag

    def _tensors(self):
        """name -> tensor of everything a checkpoint has to hold."""
        out = {}
        for name, table in (("stats", self.stats), ("precs", self.precs)):
            for order, q in table.items():
                self._store_tensors(f"{name}.{order}", q, out)
        return out

    def state_dict(self):
        return {"active": torch.tensor(self.active), **self._tensors()}

    def load_state_dict(self, sd):
        active = sd["active"]
        if torch.is_tensor(active) and active.dim() == 1:
            self.active = [bool(a) for a in active.tolist()]
        else:                                                       # one flag for the whole bank
            self.active = [bool(active)] * len(self.params)
        for name, t in self._tensors().items():
            t.copy_(sd[name])
