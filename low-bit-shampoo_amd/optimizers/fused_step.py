"""One optimizer step with the preconditioner work of all eligible parameters batched in a
ShampooBank (no counterpart in the reference, whose step() walks the parameters one by one:
optimizers/shampoo1.py:371-427, shampoo2.py:412-468), and the checkpointing of that bank."""
import math

import torch

from optimizers.shampoo_common import CODE


class _FusedStep:
    """fused=True (not in the reference) runs all eligible GPU parameters through one batched
    ShampooBank instead of one Preconditioner object per parameter; the arithmetic is the same.

    Step semantics are the reference's (optimizers/shampoo2.py:412-468, shampoo1.py:371-427): a parameter without a
    gradient is skipped -- nothing of its state moves -- and state['step'] counts per parameter, so the schedules
    (stat_compute_steps, prec_compute_steps, start_prec_step) and AdamW's bias corrections follow each parameter's
    own count.  All fp32 GPU parameters of a group that have a matrix view form the bank, whether or not they have
    a gradient at the first step; a step in which the banked parameters are at different counts works on the
    parameters that are due (per-block skip flags, or the due rows of a stack gathered, updated and put back).

    Checkpoints: state_dict() carries, next to torch's usual entries, 'shampoo_bank': one
    dict of plain tensors per parameter group -- per block order n the stacked 4/8-bit
    preconditioners ('precs.n.codes' uint8 [count, ceil(n*n*bits/8)] with the first element of a pair in
    the high nibble, 'precs.n.absmax' fp32 [count, n*ceil(n/blocksize)], 'precs.n.diag' fp32 [count, n];
    'precs.n.dense' fp32 [count, n, n] instead for orders kept in fp32) and statistics (shampoo1: the same
    under 'stats.n.'; shampoo2: 'basis.n.codes', 'basis.n.absmax' (or 'basis.n.dense'),
    'basis.n.svalue' fp32 [count, n/2], 'basis.n.keep' int64 [count, n/2],
    'basis.n.max_eigenvalue' fp32 [count], 'low_rank' int64 [orders, 3]), 'active' bool [parameters],
    'block_table' int64 [statistics, 5] = (parameter index in the bank, block index within the parameter,
    side, order, row in that order's stack).  Parameters outside the bank (non-fp32 tensors, vectors) keep
    a per-parameter preconditioner, written in its flat form under 'shampoo_preconditioners'.  Nothing in a
    checkpoint is a pickled Python object: torch.load(..., weights_only=True) reads all of it.  A checkpoint with
    'shampoo_bank' can only be loaded into an optimizer built with fused=True (ValueError otherwise: the banked
    parameters have no per-parameter preconditioner state)."""

    _update = None                 # _adamw_update or _sgd_update
    bank_keys = ()                 # group entries handed to the bank besides the common ones
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
            pending = self._pending_bank_state or []
            for index, group in enumerate(self.param_groups):
                entry = self.__dict__.get('_fused_cache', {}).get(id(group))
                if entry is None:                                 # (a loaded state that no step has consumed yet is passed on)
                    banks.append(pending[index] if index < len(pending) else None)
                    continue
                one = {}
                if entry['bank'] is not None:
                    one.update(entry['bank'].state_dict())
                    one['block_table'] = torch.tensor(entry['bank'].block_table(), dtype=torch.int64)
                banks.append(one)
            sd['shampoo_bank'] = banks
        return sd

    def load_state_dict(self, state_dict):
        state_dict = dict(state_dict)
        banks = state_dict.pop('shampoo_bank', None)
        if banks is not None and any(b for b in banks) and not self._fused:
            raise ValueError("this checkpoint was written by an optimizer with fused=True (it carries 'shampoo_bank'); "
                             "load it into an optimizer constructed with fused=True")
        super().load_state_dict(state_dict)
        if banks is not None:
            self.__dict__.pop('_fused_cache', None)          # rebuilt, then filled, by the next step
            self._pending_bank_state = list(banks)              # consumed group by group; the caller's list stays as it is


def _entry_for(opt, group, group_index):
    """The group's bank (built at the first step that finds a gradient in the group) and its bookkeeping."""
    cache = opt.__dict__.setdefault('_fused_cache', {})
    entry = cache.get(id(group))
    if entry is not None:
        return entry
    ShampooBank = opt.bank_class()
    keys = ('prec_maxorder', 'prec_bits', 'min_lowbit_size', 'quan_blocksize')
    banked = [p for p in group['params'] if ShampooBank.accepts(p, *(group[k] for k in keys))]
    bank = ShampooBank(banked, opt.name2qmap, CODE, stat_decay=group['stat_decay'], matrix_eps=group['matrix_eps'],
                       **{k: group[k] for k in keys + tuple(opt.bank_keys)}) if banked else None
    entry = cache[id(group)] = dict(bank=bank, banked=banked, index={id(p): i for i, p in enumerate(banked)})
    pending = getattr(opt, '_pending_bank_state', None)
    if pending is not None and group_index < len(pending) and pending[group_index]:
        saved = pending[group_index]
        if bank is not None:
            table = torch.tensor(bank.block_table(), dtype=torch.int64)
            if 'block_table' not in saved or not torch.equal(saved['block_table'].cpu(), table):
                raise ValueError("checkpoint was written for other parameter shapes or block sizes")
            bank.load_state_dict(saved)
        pending[group_index] = None
    return entry


def fused_step(opt, group, update, group_index=0):
    """One optimizer step of a parameter group with the preconditioner work batched."""
    params = [p for p in group['params'] if p.grad is not None]
    if not params:
        return
    for p in params:
        if p.grad.is_sparse:
            raise RuntimeError('Shampoo does not support sparse yet')
    entry = _entry_for(opt, group, group_index)
    bank, banked, index = entry['bank'], entry['banked'], entry['index']
    for p in params:                                                  # every parameter counts its own steps
        state = opt.state[p]
        state['step'] = state.get('step', 0) + 1
        if id(p) not in index and 'preconditioner' not in state:
            state['preconditioner'] = opt._make_preconditioner(p, group)
    grads = {id(p): p.grad.contiguous() for p in params}
    directions, grafted = {}, set()
    if bank is not None:
        present = [i for i, p in enumerate(banked) if p.grad is not None]
        count = {i: opt.state[banked[i]]['step'] for i in present}
        due_stats = [i for i in present if count[i] % group['stat_compute_steps'] == 0]
        due_roots = [i for i in present if count[i] % group['prec_compute_steps'] == 0]
        due_apply = [i for i in present if count[i] >= group['start_prec_step'] and (bank.active[i] or i in due_roots)]
        bgrads = [grads.get(id(p)) for p in banked]
        applied = None
        if opt.overlap_precondition and due_stats and not due_roots and due_apply and hasattr(bank, 'alongside'):
            applied = []
            bank.prepare(bgrads, only=present)                      # address tables: written once, by this thread
            bank.alongside = lambda: applied.extend(bank.preconditioned_grads(bgrads, inline=True, only=due_apply))
        if due_stats:
            bank.add_statistics(bgrads, only=due_stats)
        if due_roots:
            bank.compute_preconditioners(only=due_roots)
        if due_apply:
            # the rescaling to each gradient's norm happens inside the fused update
            if applied is None:
                applied = bank.preconditioned_grads(bgrads, only=due_apply)
            directions = {id(banked[i]): applied[i] for i in due_apply}
            grafted = set(directions)
    for p in params:
        if id(p) not in index:
            # into a buffer that stays where it is: the fused update keeps a device table of addresses
            d = opt._shampoo_direction(p, grads[id(p)], group, opt.state[p])
            kept = entry.setdefault('directions', {})
            if id(p) not in kept or kept[id(p)].shape != d.shape or kept[id(p)].dtype != d.dtype:
                kept[id(p)] = torch.empty_like(d, memory_format=torch.contiguous_format)
            directions[id(p)] = kept[id(p)].copy_(d)
    update(opt, group, params, [directions.get(id(p), grads[id(p)]) for p in params], [grads[id(p)] for p in params],
           [id(p) in grafted for p in params], [opt.state[p]['step'] for p in params], entry)


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


def _adamw_update(opt, group, params, dirs, grads, graft, steps, entry):
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
        plan.adamw(params, dirs, grads, m, v, graft, group['lr'], (beta1, beta2), group['eps'], group['weight_decay'], steps)
        return
    _graft(dirs, grads, graft)
    torch._foreach_mul_(params, 1 - group['lr'] * group['weight_decay'])
    torch._foreach_mul_(m, beta1)
    torch._foreach_add_(m, dirs, alpha=1 - beta1)
    torch._foreach_mul_(v, beta2)
    torch._foreach_addcmul_(v, dirs, dirs, value=1 - beta2)
    denom = torch._foreach_sqrt(v)
    for p, one, mom, step in zip(params, denom, m, steps):          # bias corrections follow each parameter's own count
        one.div_(math.sqrt(1 - beta2 ** step)).add_(group['eps'])
        p.addcdiv_(mom, one, value=-group['lr'] / (1 - beta1 ** step))


def _sgd_update(opt, group, params, dirs, grads, graft, steps, entry):
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


