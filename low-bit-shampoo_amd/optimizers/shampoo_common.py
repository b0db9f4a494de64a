"""Pieces shared by the two Shampoo variants: block partitioning, the per-parameter
preconditioner and the SGD / AdamW shells.

Interfaces follow the reference's optimizers/shampoo1.py and shampoo2.py (BlockPartitioner
:35-99, Preconditioner :102-244 / :102-275, ShampooSGD :247-331 / :278-367, ShampooAdamW
:334-427 / :370-468): same class and method names, constructor arguments, defaults and update
rules.  On a GPU the statistics update and the application of the preconditioners run through
the fused matrix-core kernels of qtensor.fused whenever the quantization layout allows it.
"""
import itertools
import math

import numpy as np
import torch
import torch.optim as optim

import qtensor.functional as F
from optimizers.matrix_functions import ComputePower, ComputePowerBatched
from qtensor.utils import QTensorDiagReal

CODE = 'linear-2'


class BlockPartitioner:
    """Cuts every dimension longer than block_size into pieces of block_size (last piece
    shorter) and lists the square preconditioner shapes, one per piece and dimension, in
    row-major order of the pieces."""

    def __init__(self, var, block_size):
        self._shape = var.shape
        self._splits = []          # (dim, cut positions) for every dimension that is cut
        self._split_sizes = []     # (dim, piece sizes)
        per_dim = []
        for dim, extent in enumerate(var.shape):
            if block_size > 0 and extent > block_size:
                cuts = (extent - 1) // block_size
                positions = (np.arange(cuts, dtype=np.int32) + 1) * block_size
                sizes = np.full(cuts + 1, block_size, dtype=np.int32)
                sizes[-1] = extent - positions[-1]
                self._splits.append((dim, positions))
                self._split_sizes.append((dim, sizes))
                per_dim.append(sizes)
            else:
                per_dim.append(np.array([extent], dtype=np.int32))
        self._num_splits = len(per_dim)
        self._preconditioner_shapes = []
        for combo in itertools.product(*per_dim):
            self._preconditioner_shapes.extend([[d, d] for d in combo])

    def shapes_for_preconditioners(self):
        return self._preconditioner_shapes

    def num_splits(self):
        return self._num_splits

    def partition(self, tensor):
        """List of block views, row-major over the pieces."""
        assert tensor.shape == self._shape
        blocks = [tensor]
        for dim, sizes in self._split_sizes:
            blocks = [piece for t in blocks for piece in torch.split(t, tuple(int(s) for s in sizes), dim=dim)]
        return blocks

    def merge_partitions(self, partitions):
        """Inverse of partition."""
        for dim, positions in reversed(self._splits):
            n = len(positions) + 1
            partitions = [torch.cat(partitions[i:i + n], axis=dim) for i in range(0, len(partitions), n)]
        assert len(partitions) == 1
        return partitions[0]


def _fusable(holder) -> bool:
    """True when a holder is low-bit on a GPU in the layout the fused kernels read directly."""
    return (holder.bits < 16 and holder.var.is_cuda and holder.var_order % holder.blocksize == 0
            and holder.var_dtype == torch.float32)


class PreconditionerBase:
    """Statistics and preconditioners of one parameter.

    The parameter is viewed as a matrix (first dimension x everything else, 1-sized dimensions
    dropped), cut into blocks of at most prec_maxorder per side; every block owns a left and a
    right statistic and preconditioner.  Low-bit storage is used on accelerators only
    (reference: shampoo1.py:125-128): on the CPU everything stays in fp32."""

    def __init__(self, var, name2qmap, stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1200,
                 prec_bits=32, min_lowbit_size=4096, quan_blocksize=64, **extra):
        self.stat_decay = stat_decay
        self.matrix_eps = matrix_eps
        self._original_shape = var.shape
        self._transformed_shape = [x for x in var.shape if x != 1]
        if len(self._transformed_shape) > 1:
            self._transformed_shape = (self._transformed_shape[0], -1)
        as_matrix = torch.reshape(var, self._transformed_shape)
        self._partitioner = BlockPartitioner(as_matrix, prec_maxorder)
        shapes = self._partitioner.shapes_for_preconditioners()
        rank = len(self._transformed_shape)
        on_accelerator = var.is_cuda or var.device.type == 'mps'
        bits = prec_bits if on_accelerator else 32
        self._active = False
        self._warned_null_preconditioner = False
        self.statistics, self.preconditioners = [], []
        if rank <= 1:
            return
        quant_args = dict(bits=bits, name2qmap=name2qmap, code=CODE, blocksize=quan_blocksize,
                          min_lowbit_size=min_lowbit_size)
        for index, (order, _) in enumerate(shapes):
            self.statistics.append(self._new_statistic(order, var.device, index, rank, quant_args, extra))
        self.preconditioners = [QTensorDiagReal(torch.eye(order, device=var.device), **quant_args)
                                for order, _ in shapes]

    # ---- hooks of the two variants ----
    def _new_statistic(self, order, device, index, rank, quant_args, extra):
        raise NotImplementedError

    def _accumulate(self, holder, block, axis, w1, w2):
        raise NotImplementedError

    def _inverse_root(self, holder, exp, eps):
        raise NotImplementedError

    # ---- reference interface ----
    def set_device(self, device):
        if len(self._transformed_shape) <= 1:
            return
        for holder in self.statistics + self.preconditioners:
            holder.set_device(device)

    def add_statistics(self, grad):
        """Fold the Gram matrices of the gradient blocks into the statistics:
        L <- w1 L + w2 G G^T, R <- w1 R + w2 G^T G."""
        if not self.statistics:
            return
        blocks = self._partitioner.partition(torch.reshape(grad, self._transformed_shape))
        w1 = self.stat_decay
        w2 = 1.0 if w1 == 1.0 else (1.0 - w1)
        rank = len(self._transformed_shape)
        for j, block in enumerate(blocks):
            block = block.float()
            for axis in range(rank):
                self._accumulate(self.statistics[j * rank + axis], block, axis, w1, w2)

    def compute_preconditioners(self, v0=None):
        """Refresh every preconditioner with the inverse 4th root of its statistic.
        v0 (not in the reference): optional start vectors of the power iteration, one per
        statistic; by default they are drawn from the global generator as the reference does."""
        for i, (stat, prec) in enumerate(zip(self.statistics, self.preconditioners)):
            self._v0 = None if v0 is None else v0[i]
            prec.quantize(self._inverse_root(stat, 4, self.matrix_eps))
        self._v0 = None
        self._active = True

    def preconditioned_grad(self, grad):
        """P_L G P_R for every block, merged back into the gradient's shape."""
        if not self.preconditioners:
            return grad
        blocks = self._partitioner.partition(torch.reshape(grad, self._transformed_shape))
        per_block = self._partitioner.num_splits()
        outs = []
        for i, block in enumerate(blocks):
            factors = self.preconditioners[i * per_block:(i + 1) * per_block]
            if (block.dim() == 2 and block.is_cuda and block.dtype == torch.float32
                    and all(_fusable(f) for f in factors)):
                from qtensor import fused as X
                outs.append(X.precondition(block, X.Quantized.from_holder(factors[0]), X.Quantized.from_holder(factors[1])))
                continue
            out = block
            for j in range(block.dim()):
                P = factors[j].dequantize().to(block.dtype)
                if block.dim() == 2 and _own_products(P, out):
                    from qtensor import fused as X
                    out = X.gemm(out, P) if j == 1 else X.gemm(P, out)
                else:
                    out = out @ P if j == 1 else P @ out
            outs.append(out)
        return torch.reshape(self._partitioner.merge_partitions(outs), self._original_shape)

    def is_active(self) -> bool:
        return self._active

    # ---- flat checkpoint form (the reference pickles this object: optimizers/shampoo2.py:311-317) ----
    def state_dict(self):
        """Plain tensors, numbers and lists only (readable with torch.load(weights_only=True)): 'active' and,
        per block and side in the order of BlockPartitioner.shapes_for_preconditioners(), the holders'
        own state_dict()s under 'statistics' and 'preconditioners'."""
        return {"active": bool(self._active),
                "statistics": [h.state_dict() for h in self.statistics],
                "preconditioners": [h.state_dict() for h in self.preconditioners]}

    def load_state_dict(self, sd):
        if len(sd["statistics"]) != len(self.statistics) or len(sd["preconditioners"]) != len(self.preconditioners):
            raise ValueError("checkpoint was written for another parameter shape or block size")
        self._active = bool(sd["active"])
        for holder, one in zip(self.statistics, sd["statistics"]):
            holder.load_state_dict(one)
        for holder, one in zip(self.preconditioners, sd["preconditioners"]):
            holder.load_state_dict(one)


def _own_products(*tensors) -> bool:
    """fp32 GPU matrices go through the library's matrix-core products instead of torch's."""
    from qtensor import fused as X
    return all(t.dim() == 2 for t in tensors) and X.on_matrix_cores(*tensors)


def dense_gram(block, axis):
    if _own_products(block):
        from qtensor import fused as X
        return X.gram(block, 0 if axis == 0 else 1)
    return block.T @ block if axis == 1 else block @ block.T


def decay_and_add_gram(stat, block, axis, w1, w2):
    """stat <- w1 * stat + w2 * (block block^T or block^T block), in place (reference: tensor.mul_(w1).add_(gram, alpha=w2),
    optimizers/shampoo1.py:164-178); one launch on the matrix cores for fp32 GPU matrices."""
    if _own_products(block, stat):
        from qtensor import fused as X
        return X.gram(block, 0 if axis == 0 else 1, stat=stat, beta=w1, alpha=w2, out=stat)
    return stat.mul_(w1).add_(dense_gram(block, axis), alpha=w2)


def newton_inverse_root(mat, exp, eps, v0=None):
    """(mat + ridge)^(-1/exp) by the coupled Newton iteration; matrix cores on a GPU."""
    mat = mat.float()
    if mat.is_cuda and F.lib is not None and mat.dim() == 2 and mat.shape[0] > 1:
        start = None if v0 is None else v0.reshape(1, -1)
        return ComputePowerBatched(mat.unsqueeze(0).contiguous(), exp, ridge_epsilon=eps, v0=start)[0]
    return ComputePower(mat, exp, ridge_epsilon=eps, v0=v0)


def build_code_maps(prec_bits):
    maps = {}
    if prec_bits in (4, 8):
        if CODE == 'dynamic':
            maps[CODE] = F.create_dynamic_map(signed=True, total_bits=prec_bits, power=1)
        elif CODE == 'linear-2':
            maps[CODE] = F.create_linear_map(signed=True, total_bits=prec_bits, power=2)
    return maps


_PREC_KEYS = ('stat_decay', 'matrix_eps', 'prec_maxorder', 'prec_bits', 'min_lowbit_size', 'quan_blocksize')


class _ShampooOptimizer(optim.Optimizer):
    """Common machinery of the SGD and AdamW shells."""
    preconditioner_class = None
    extra_keys = ()

    def _init_shampoo(self, prec_bits):
        self.name2qmap = build_code_maps(prec_bits)

    def state_dict(self):
        """torch's layout, except that no Python object is pickled: the per-parameter preconditioners leave the
        'state' entries and go, in their flat form (PreconditionerBase.state_dict: tensors, numbers, lists), to
        'shampoo_preconditioners' = {parameter id as in 'state': flat dict}.  (The reference leaves the
        Preconditioner objects in the state and thus in the pickle: optimizers/shampoo2.py:311-317.)"""
        sd = super().state_dict()
        flat, state = {}, {}
        for pid, one in sd['state'].items():
            prec = one.get('preconditioner') if isinstance(one, dict) else None
            if isinstance(prec, PreconditionerBase):
                flat[pid] = prec.state_dict()
                one = {k: v for k, v in one.items() if k != 'preconditioner'}
            state[pid] = one
        sd['state'] = state
        sd['shampoo_preconditioners'] = flat
        return sd

    def load_state_dict(self, state_dict):
        """Reads what state_dict() writes; a checkpoint whose 'state' entries still hold Preconditioner objects
        (the reference's form) is taken as well."""
        state_dict = dict(state_dict)
        flat = state_dict.pop('shampoo_preconditioners', None) or {}
        super().load_state_dict(state_dict)
        by_id = {}
        for group, saved in zip(self.param_groups, state_dict['param_groups']):
            for p, pid in zip(group['params'], saved['params']):
                by_id[pid] = (p, group)
        for pid, one in flat.items():
            p, group = by_id[pid]
            prec = self._make_preconditioner(p, group)
            prec.load_state_dict(one)
            self.state[p]['preconditioner'] = prec
        for group in self.param_groups:
            for p in group['params']:
                state = self.state[p]
                if len(state) != 0 and isinstance(state.get('preconditioner'), PreconditionerBase):
                    state['preconditioner'].set_device(p.device)

    def _make_preconditioner(self, p, group):
        kwargs = {k: group[k] for k in _PREC_KEYS + tuple(self.extra_keys)}
        return self.preconditioner_class(p, self.name2qmap, **kwargs)

    def _shampoo_direction(self, p, grad, group, state, statistics_done=False, roots_done=False):
        """Statistics / inverse-root bookkeeping for this step and the grafted direction
        (statistics_done / roots_done: the caller has already run this step's add_statistics /
        compute_preconditioners)."""
        prec = state['preconditioner']
        if state['step'] % group['stat_compute_steps'] == 0 and not statistics_done:
            prec.add_statistics(grad)
        if state['step'] % group['prec_compute_steps'] == 0 and not roots_done:
            prec.compute_preconditioners()
        direction = grad
        if state['step'] >= group['start_prec_step'] and prec.is_active():
            direction = prec.preconditioned_grad(grad)
            direction.mul_(grad.norm() / (direction.norm() + 1e-12))      # keep the gradient's norm
        return direction


class ShampooSGDBase(_ShampooOptimizer):
    def __init__(self, params, lr=0.1, momentum=0.9, weight_decay=0.0, nesterov=False, start_prec_step=1,
                 stat_compute_steps=100, prec_compute_steps=500, stat_decay=0.95, matrix_eps=1e-6,
                 prec_maxorder=1200, prec_bits=32, min_lowbit_size=4096, quan_blocksize=64, **extra):
        defaults = dict(lr=lr, momentum=momentum, weight_decay=weight_decay, nesterov=nesterov,
                        start_prec_step=start_prec_step, stat_compute_steps=stat_compute_steps,
                        prec_compute_steps=prec_compute_steps, stat_decay=stat_decay, matrix_eps=matrix_eps,
                        prec_maxorder=prec_maxorder, prec_bits=prec_bits, min_lowbit_size=min_lowbit_size,
                        quan_blocksize=quan_blocksize, **extra)
        super().__init__(params, defaults)
        self._init_shampoo(prec_bits)

    @torch.no_grad()
    def step(self, closure=None):
        for group in self.param_groups:
            for p in group['params']:
                if p.grad is None:
                    continue
                grad = p.grad.data
                if grad.is_sparse:
                    raise RuntimeError('Shampoo does not support sparse yet')
                state = self.state[p]
                if len(state) == 0:
                    state['step'] = 0
                    state['preconditioner'] = self._make_preconditioner(p, group)
                    state['momentum'] = torch.zeros_like(p, memory_format=torch.preserve_format)
                state['step'] += 1
                direction = self._shampoo_direction(p, grad, group, state)
                if group['weight_decay'] != 0.0:
                    direction.add_(p.data, alpha=group['weight_decay'])
                buf = state['momentum'].mul_(group['momentum']).add_(direction)
                update = direction.add(buf, alpha=group['momentum']) if group['nesterov'] else buf
                p.data.add_(update, alpha=-group['lr'])


class ShampooAdamWBase(_ShampooOptimizer):
    def __init__(self, params, lr=0.001, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, start_prec_step=1,
                 stat_compute_steps=100, prec_compute_steps=500, stat_decay=0.95, matrix_eps=1e-6,
                 prec_maxorder=1200, prec_bits=32, min_lowbit_size=4096, quan_blocksize=64, **extra):
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, start_prec_step=start_prec_step,
                        stat_compute_steps=stat_compute_steps, prec_compute_steps=prec_compute_steps,
                        stat_decay=stat_decay, matrix_eps=matrix_eps, prec_maxorder=prec_maxorder,
                        prec_bits=prec_bits, min_lowbit_size=min_lowbit_size, quan_blocksize=quan_blocksize, **extra)
        super().__init__(params, defaults)
        self._init_shampoo(prec_bits)

    @torch.no_grad()
    def step(self, closure=None):
        for group in self.param_groups:
            for p in group['params']:
                if p.grad is None:
                    continue
                grad = p.grad.data
                if grad.is_sparse:
                    raise RuntimeError('Shampoo does not support sparse yet')
                state = self.state[p]
                if len(state) == 0:
                    state['step'] = 0
                    state['preconditioner'] = self._make_preconditioner(p, group)
                    state['exp_avg'] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    state['exp_avg_sq'] = torch.zeros_like(p, memory_format=torch.preserve_format)
                state['step'] += 1
                p.mul_(1 - group['lr'] * group['weight_decay'])           # decoupled weight decay
                direction = self._shampoo_direction(p, grad, group, state)
                beta1, beta2 = group['betas']
                correction1 = 1 - beta1 ** state['step']
                correction2 = 1 - beta2 ** state['step']
                m, v = state['exp_avg'], state['exp_avg_sq']
                m.mul_(beta1).add_(direction, alpha=1 - beta1)
                v.mul_(beta2).addcmul_(direction, direction, value=1 - beta2)
                denom = (v.sqrt() / math.sqrt(correction2)).add_(group['eps'])
                p.addcdiv_(m, denom, value=-group['lr'] / correction1)


_DOC = r"""
    {base} with Shampoo preconditioning of every parameter that has a matrix view.

    Arguments beyond those of {base} (names and defaults as in the reference's optimizers):
        start_prec_step: first step at which the preconditioned direction is used
        stat_compute_steps: T_1, the statistics L, R take in a gradient every T_1-th step
        prec_compute_steps: T_2, the inverse 4th roots are recomputed every T_2-th step
        stat_decay: beta of L <- beta L + (1 - beta) G G^T (1.0: plain sum)
        matrix_eps: epsilon, the initial statistic is epsilon I and the ridge is epsilon times the largest eigenvalue
        prec_maxorder: sides longer than this are cut into blocks of at most this order
        prec_bits: 32, 16, 8 or 4, the storage width of statistics and preconditioners
        min_lowbit_size: matrices with fewer elements stay in fp32 whatever prec_bits says
        quan_blocksize: elements per quantization segment (64 ... 2048){more}
    """
