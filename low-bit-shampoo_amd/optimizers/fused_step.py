"""One optimizer step with the preconditioner work of all eligible parameters batched in a
ShampooBank (no counterpart in the reference, whose step() walks the parameters one by one:
optimizers/shampoo1.py:371-427, shampoo2.py:412-468), and the checkpointing of that bank."""
import torch

from optimizers.engine import UNBATCHED_SLOT as _UNBATCHED_SLOT, SideJob as _SideJob, shared_stream as _shared_stream
from optimizers.shampoo_common import CODE


class _FusedStep:
    """fused=True (not in the reference) runs all eligible GPU parameters through one batched
    ShampooBank instead of one Preconditioner object per parameter; the arithmetic is the same.

    Differences from the reference's step(), which walks the parameters one by one and skips those without a
    gradient (optimizers/shampoo1.py:371-377): the parameters that have a gradient at the first step form the bank,
    and every one of them needs a gradient at every later step (RuntimeError otherwise); state['step'] is the
    group's step count for every parameter, so a parameter that first gets a gradient later shares the group's
    bias corrections and schedules.

    Checkpoints: state_dict() then carries, next to torch's usual entries, 'shampoo_bank': one
    dict of plain tensors per parameter group -- per block order n the stacked 4/8-bit
    preconditioners ('precs.n.codes' uint8 [count, n*n*bits/8] with the first element of a pair in
    the high nibble, 'precs.n.absmax' fp32 [count, n*n/blocksize], 'precs.n.diag' fp32 [count, n])
    and statistics (shampoo1: the same three under 'stats.n.'; shampoo2: 'basis.n.codes',
    'basis.n.absmax', 'basis.n.svalue' fp32 [count, n/2], 'basis.n.keep' int64 [count, n/2],
    'basis.n.max_eigenvalue' fp32 [count]), 'block_table' int64 [statistics, 5] = (parameter index
    in the group, block index within the parameter, side, order, row in that order's stack), and
    the step count.  Nothing in 'shampoo_bank' is a pickled Python object, so torch.load(..., weights_only=True) reads
    that part; parameters outside the bank (an order that the blocksize does not divide, non-fp32 tensors) keep the
    reference's state['preconditioner'] object in the usual per-parameter state, which needs weights_only=False like
    the reference's own checkpoints.  A checkpoint with 'shampoo_bank' can only be loaded into an optimizer built with
    fused=True (ValueError otherwise: the banked parameters have no per-parameter preconditioner state)."""

    _update = None                 # _adamw_update or _sgd_update
    bank_keys = ()                 # group entries handed to the bank besides the common ones
    # True: the statistics update of the parameters the bank does not take runs on a thread of its own while
    # the bank updates its statistics (worth it where that update waits for the device again and again)
    overlap_unbatched_statistics = False
    # True: the inverse roots of those parameters (a Newton iteration that waits for the device twice per round)
    # are computed on a thread of their own while the bank's batched iteration runs; their power-iteration start
    # vectors are then drawn first, on the calling thread, so that the generator is used in a fixed order
    overlap_unbatched_inverse_roots = True
    # True: on steps that update the statistics and keep the inverse roots, the bank applies the stored roots to
    # the gradients on a thread and a stream of its own while the factorisations of the statistics update run
    # (chains of small launches that leave part of the device waiting; the two read the same gradients and
    # share nothing else).  Needs a bank whose add_statistics runs the callable it finds in bank.alongside.
    overlap_precondition = False

    @staticmethod
    def bank_class():
        from optimizers.engine import ShampooBank
        return ShampooBank

    def _init_fused(self, fused):
        self._fused = fused
        self._pending_bank_state = None

    @torch.no_grad()
    def step(self, closure=None):
        if not self._fused:
            return super().step(closure)
        for index, group in enumerate(self.param_groups):
            fused_step(self, group, type(self)._update, index)

    def state_dict(self):
        sd = super().state_dict()
        if self._fused:
            banks = []
            for group in self.param_groups:
                entry = self.__dict__.get('_fused_cache', {}).get(id(group))
                if entry is None:
                    banks.append(None)
                    continue
                one = {'step': torch.tensor(entry['step'])}
                if entry['bank'] is not None:
                    one.update(entry['bank'].state_dict())
                    one['block_table'] = torch.tensor(entry['bank'].block_table(), dtype=torch.int64)
                banks.append(one)
            sd['shampoo_bank'] = banks
        return sd

    def load_state_dict(self, state_dict):
        state_dict = dict(state_dict)
        banks = state_dict.pop('shampoo_bank', None)
        if banks is not None and any(b is not None for b in banks) and not self._fused:
            raise ValueError("this checkpoint was written by an optimizer with fused=True (it carries 'shampoo_bank'); "
                             "load it into an optimizer constructed with fused=True")
        super().load_state_dict(state_dict)
        if banks is not None:
            self.__dict__.pop('_fused_cache', None)          # rebuilt, then filled, by the next step
            self._pending_bank_state = list(banks)              # consumed group by group; the caller's list stays as it is


def fused_step(opt, group, update, group_index=0):
    """One optimizer step of a parameter group with the preconditioner work batched."""
    ShampooBank = opt.bank_class()

    params = [p for p in group['params'] if p.grad is not None]
    if not params:
        return
    cache = opt.__dict__.setdefault('_fused_cache', {})
    entry = cache.get(id(group))
    if entry is None:
        keys = ('prec_maxorder', 'prec_bits', 'min_lowbit_size', 'quan_blocksize')
        banked = [p for p in params if ShampooBank.accepts(p, *(group[k] for k in keys))]
        bank = ShampooBank(banked, opt.name2qmap, CODE, stat_decay=group['stat_decay'], matrix_eps=group['matrix_eps'],
                           **{k: group[k] for k in keys + tuple(opt.bank_keys)}) if banked else None
        entry = cache[id(group)] = dict(bank=bank, banked=banked, ids={id(p) for p in banked}, step=0)
        for p in params:
            state = opt.state[p]
            state.setdefault('step', 0)
            if id(p) not in entry['ids'] and 'preconditioner' not in state:
                state['preconditioner'] = opt._make_preconditioner(p, group)
        pending = getattr(opt, '_pending_bank_state', None)
        if pending is not None and group_index < len(pending) and pending[group_index] is not None:
            saved = pending[group_index]
            entry['step'] = int(saved['step'])
            if bank is not None:
                table = torch.tensor(bank.block_table(), dtype=torch.int64)
                if 'block_table' not in saved or not torch.equal(saved['block_table'].cpu(), table):
                    raise ValueError("checkpoint was written for other parameter shapes or block sizes")
                bank.load_state_dict(saved)
            pending[group_index] = None
    if any(p.grad is None for p in entry['banked']):                  # before anything of this step is counted or launched
        raise RuntimeError("fused=True batches the parameters that had a gradient at the first step; "
                           "every one of them needs a gradient at every later step")
    entry['step'] += 1
    step, bank, banked = entry['step'], entry['bank'], entry['banked']
    for p in params:
        state = opt.state[p]
        state['step'] = step
        if id(p) not in entry['ids'] and 'preconditioner' not in state:      # first gradient after the bank was built
            state['preconditioner'] = opt._make_preconditioner(p, group)
    grads = {id(p): p.grad.contiguous() for p in params}
    directions, grafted = {}, set()
    unbatched = [p for p in params if id(p) not in entry['ids']]
    side_job, roots_done, statistics_done = None, False, False
    if (bank is not None and unbatched and opt.overlap_unbatched_statistics and step % group['stat_compute_steps'] == 0
            and all('preconditioner' in opt.state[p] for p in unbatched)):
        if entry.get('side_stream') is None:
            entry['side_stream'] = _shared_stream(unbatched[0].device, _UNBATCHED_SLOT)

        def update_unbatched():
            for q in unbatched:
                opt.state[q]['preconditioner'].add_statistics(grads[id(q)])

        side_job = _SideJob(unbatched[0].device, entry['side_stream'], update_unbatched)
    if bank is not None:
        bgrads = [grads[id(p)] for p in banked]
        applied = None
        if (opt.overlap_precondition and step % group['stat_compute_steps'] == 0 and step % group['prec_compute_steps'] != 0
                and step >= group['start_prec_step'] and bank.is_active() and hasattr(bank, 'alongside')):
            applied = []
            bank.prepare(bgrads)                                       # address tables: written once, by this thread
            bank.alongside = lambda: applied.extend(bank.preconditioned_grads(bgrads, inline=True))
        if step % group['stat_compute_steps'] == 0:
            try:
                bank.add_statistics(bgrads)
            finally:
                if side_job is not None:
                    side_job.join()
                    statistics_done = True
        if step % group['prec_compute_steps'] == 0:
            roots_job = None
            if (unbatched and opt.overlap_unbatched_inverse_roots
                    and all('preconditioner' in opt.state[p] for p in unbatched)):
                if entry.get('side_stream') is None:
                    entry['side_stream'] = _shared_stream(unbatched[0].device, _UNBATCHED_SLOT)
                if side_job is None and step % group['stat_compute_steps'] == 0:
                    for q in unbatched:                               # this step's statistics come before its roots
                        opt.state[q]['preconditioner'].add_statistics(grads[id(q)])
                    statistics_done = True
                draw = group.get('inv_root_mode', 1) != 0              # the eigenpair route uses no start vectors
                starts = {id(q): [torch.rand(h.var_order, device=q.device) * 2 - 1
                                  for h in opt.state[q]['preconditioner'].statistics] if draw else None
                          for q in unbatched}

                def roots_of_unbatched():
                    for q in unbatched:
                        opt.state[q]['preconditioner'].compute_preconditioners(v0=starts[id(q)])

                roots_job = _SideJob(unbatched[0].device, entry['side_stream'], roots_of_unbatched)
        else:
            roots_job = None
        try:
            if step % group['prec_compute_steps'] == 0:
                bank.compute_preconditioners()
            if step >= group['start_prec_step'] and bank.is_active():
                # the rescaling to each gradient's norm happens inside the fused update
                if applied is None:
                    applied = bank.preconditioned_grads(bgrads)
                directions = {id(p): o for p, o in zip(banked, applied)}
                grafted = set(directions)
        finally:
            # (joined behind the bank's products with the new roots: the current stream waits for the small launches
            # of the side job only where the parameters outside the bank need their roots)
            if roots_job is not None:
                roots_job.join()
                roots_done = True
    for p in params:
        if id(p) not in entry['ids']:
            # into a buffer that stays where it is: the fused update keeps a device table of addresses
            d = opt._shampoo_direction(p, grads[id(p)], group, opt.state[p], statistics_done=statistics_done,
                                       roots_done=roots_done)
            kept = entry.setdefault('directions', {})
            if id(p) not in kept or kept[id(p)].shape != d.shape or kept[id(p)].dtype != d.dtype:
                kept[id(p)] = torch.empty_like(d, memory_format=torch.contiguous_format)
            directions[id(p)] = kept[id(p)].copy_(d)
    update(opt, group, params, [directions.get(id(p), grads[id(p)]) for p in params], [grads[id(p)] for p in params],
           [id(p) in grafted for p in params], step, entry)


def _fused_tail_ok(params, dirs):
    return all(p.is_cuda and p.dtype == torch.float32 and p.is_contiguous() and d.dtype == torch.float32 and d.is_contiguous()
               for p, d in zip(params, dirs))


def _tail_plan(entry):
    from optimizers.tail import TailPlan
    if entry.get('tail') is None:
        entry['tail'] = TailPlan()
    return entry['tail']


def _graft(dirs, grads, graft):
    # keep each gradient's norm (reference: shampoo1.py:421)
    for d, g, f in zip(dirs, grads, graft):
        if f:
            d.mul_(g.norm() / (d.norm() + 1e-12))


def _adamw_update(opt, group, params, dirs, grads, graft, step, entry):
    import math
    for p in params:
        state = opt.state[p]
        if 'exp_avg' not in state:
            state['exp_avg'] = torch.zeros_like(p, memory_format=torch.preserve_format)
            state['exp_avg_sq'] = torch.zeros_like(p, memory_format=torch.preserve_format)
    m = [opt.state[p]['exp_avg'] for p in params]
    v = [opt.state[p]['exp_avg_sq'] for p in params]
    beta1, beta2 = group['betas']
    if _fused_tail_ok(params, dirs):
        plan = _tail_plan(entry)
        plan.adamw(params, dirs, grads, m, v, graft, group['lr'], (beta1, beta2), group['eps'], group['weight_decay'], step)
        return
    _graft(dirs, grads, graft)
    torch._foreach_mul_(params, 1 - group['lr'] * group['weight_decay'])
    torch._foreach_mul_(m, beta1)
    torch._foreach_add_(m, dirs, alpha=1 - beta1)
    torch._foreach_mul_(v, beta2)
    torch._foreach_addcmul_(v, dirs, dirs, value=1 - beta2)
    denom = torch._foreach_sqrt(v)
    torch._foreach_div_(denom, math.sqrt(1 - beta2 ** step))
    torch._foreach_add_(denom, group['eps'])
    torch._foreach_addcdiv_(params, m, denom, value=-group['lr'] / (1 - beta1 ** step))


def _sgd_update(opt, group, params, dirs, grads, graft, step, entry):
    for p in params:
        state = opt.state[p]
        if 'momentum' not in state:
            state['momentum'] = torch.zeros_like(p, memory_format=torch.preserve_format)
    bufs = [opt.state[p]['momentum'] for p in params]
    if _fused_tail_ok(params, dirs):
        plan = _tail_plan(entry)
        plan.sgd(params, dirs, grads, bufs, graft, group['lr'], group['momentum'], group['weight_decay'], group['nesterov'])
        return
    _graft(dirs, grads, graft)
    if group['weight_decay'] != 0.0:
        torch._foreach_add_(dirs, params, alpha=group['weight_decay'])
    torch._foreach_mul_(bufs, group['momentum'])
    torch._foreach_add_(bufs, dirs)
    if group['nesterov']:
        dirs = torch._foreach_add(dirs, bufs, alpha=group['momentum'])
    else:
        dirs = bufs
    torch._foreach_add_(params, dirs, alpha=-group['lr'])


