"""Low-bit Shampoo that quantizes the eigenvector matrix of each statistic instead of the
statistic itself ("ours" in the paper): every statistic is a QTensorSVDFast.

Same module surface as the reference's optimizers/shampoo2.py: BlockPartitioner,
Preconditioner, ShampooSGD, ShampooAdamW, CODE; three more constructor arguments than
shampoo1 (rect_t1, rect_t2, inv_root_mode).
"""
import itertools

import torch

from optimizers.shampoo_common import (CODE, BlockPartitioner, PreconditionerBase, ShampooAdamWBase, ShampooSGDBase,
                                       _DOC, decay_and_add_gram, newton_inverse_root)
from optimizers.fused_step import _FusedStep, _adamw_update, _sgd_update
from qtensor.utils import QTensorSVDFast

__all__ = ["CODE", "BlockPartitioner", "Preconditioner", "ShampooSGD", "ShampooAdamW"]


class Preconditioner(PreconditionerBase):
    """Compute statistics/shape from gradients for preconditioning (reference: shampoo2.py:102-275).

    inv_root_mode 0: inverse root from the stored eigenpairs (QTensorSVDFast.computepower);
    inv_root_mode 1: coupled Newton iteration on the dequantized statistic."""

    def __init__(self, var, name2qmap, stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1200,
                 prec_bits=32, min_lowbit_size=4096, quan_blocksize=64, rect_t1=1, rect_t2=4, inv_root_mode=0):
        if not hasattr(Preconditioner, '_instance_counter'):
            Preconditioner._instance_counter = itertools.count()
        self.inv_root_mode = inv_root_mode
        self._log_prefix = f"pre_{next(Preconditioner._instance_counter)}"
        super().__init__(var, name2qmap, stat_decay=stat_decay, matrix_eps=matrix_eps, prec_maxorder=prec_maxorder,
                         prec_bits=prec_bits, min_lowbit_size=min_lowbit_size, quan_blocksize=quan_blocksize,
                         rect_t1=rect_t1, rect_t2=rect_t2)

    def _new_statistic(self, order, device, index, rank, quant_args, extra):
        prefix = f"{self._log_prefix}_block{index // rank}_axis{index % rank}"
        return QTensorSVDFast(self.matrix_eps * torch.eye(order, device=device), rect_t1=extra['rect_t1'],
                              rect_t2=extra['rect_t2'], log_prefix=prefix, **quant_args)

    def _accumulate(self, holder, block, axis, w1, w2):
        # rebuild L from the kept eigenpairs, decay, add the Gram matrix, re-diagonalise
        # (reference: shampoo2.py:185-200)
        stat, basis = holder.dequantize()
        decay_and_add_gram(stat, block, axis, w1, w2)
        holder.quantize(stat, basis)

    def _inverse_root(self, holder, exp, eps):
        if self.inv_root_mode == 0:
            return holder.computepower(exp, ridge_epsilon=eps)
        stat, _ = holder.dequantize()
        return newton_inverse_root(stat, exp, eps, getattr(self, '_v0', None)).to(stat.dtype)


class _Fused2(_FusedStep):
    bank_keys = ('rect_t1', 'rect_t2', 'inv_root_mode')
    overlap_precondition = True              # the stored roots are applied to the gradients next to the factorisations

    @staticmethod
    def bank_class():
        from optimizers.engine2 import ShampooBank2
        return ShampooBank2


class ShampooSGD(_Fused2, ShampooSGDBase):
    preconditioner_class = Preconditioner
    extra_keys = ('rect_t1', 'rect_t2', 'inv_root_mode')
    _update = staticmethod(_sgd_update)

    def __init__(self, params, lr=0.1, momentum=0.9, weight_decay=0.0, nesterov=False, start_prec_step=1,
                 stat_compute_steps=100, prec_compute_steps=500, stat_decay=0.95, matrix_eps=1e-6,
                 prec_maxorder=1200, prec_bits=32, min_lowbit_size=4096, quan_blocksize=64,
                 rect_t1=1, rect_t2=4, inv_root_mode=0, fused=False):
        self._init_fused(fused)
        super().__init__(params, lr=lr, momentum=momentum, weight_decay=weight_decay, nesterov=nesterov,
                         start_prec_step=start_prec_step, stat_compute_steps=stat_compute_steps,
                         prec_compute_steps=prec_compute_steps, stat_decay=stat_decay, matrix_eps=matrix_eps,
                         prec_maxorder=prec_maxorder, prec_bits=prec_bits, min_lowbit_size=min_lowbit_size,
                         quan_blocksize=quan_blocksize, rect_t1=rect_t1, rect_t2=rect_t2, inv_root_mode=inv_root_mode)


class ShampooAdamW(_Fused2, ShampooAdamWBase):
    preconditioner_class = Preconditioner
    extra_keys = ('rect_t1', 'rect_t2', 'inv_root_mode')
    _update = staticmethod(_adamw_update)

    def __init__(self, params, lr=0.001, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, start_prec_step=1,
                 stat_compute_steps=100, prec_compute_steps=500, stat_decay=0.95, matrix_eps=1e-6,
                 prec_maxorder=1200, prec_bits=32, min_lowbit_size=4096, quan_blocksize=64,
                 rect_t1=1, rect_t2=4, inv_root_mode=0, fused=False):
        self._init_fused(fused)
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay,
                         start_prec_step=start_prec_step, stat_compute_steps=stat_compute_steps,
                         prec_compute_steps=prec_compute_steps, stat_decay=stat_decay, matrix_eps=matrix_eps,
                         prec_maxorder=prec_maxorder, prec_bits=prec_bits, min_lowbit_size=min_lowbit_size,
                         quan_blocksize=quan_blocksize, rect_t1=rect_t1, rect_t2=rect_t2, inv_root_mode=inv_root_mode)


_MORE = """
        rect_t1: Bjorck steps V <- 1.5 V - 0.5 V V^T V on the dequantized basis before a statistic is rebuilt
        rect_t2: the same before an inverse root is taken from the stored eigenpairs
        inv_root_mode: 0 = inverse root from the stored eigenpairs, 1 = coupled Newton iteration on the rebuilt statistic"""
ShampooSGD.__doc__ = _DOC.format(base="SGD", more=_MORE) + _FusedStep.__doc__
ShampooAdamW.__doc__ = _DOC.format(base="AdamW", more=_MORE) + _FusedStep.__doc__
