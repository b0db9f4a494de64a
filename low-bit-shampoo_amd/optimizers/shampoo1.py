""""Naive" low-bit Shampoo: the statistics L, R themselves are stored quantized (with an exact
diagonal) and the inverse 4th roots always come from the coupled Newton iteration.

Same module surface as the reference's optimizers/shampoo1.py: BlockPartitioner,
Preconditioner, ShampooSGD, ShampooAdamW, CODE.
"""
import torch

from optimizers.shampoo_common import (CODE, BlockPartitioner, PreconditionerBase, ShampooAdamWBase, ShampooSGDBase,
                                       _DOC, _fusable, decay_and_add_gram, newton_inverse_root)
from optimizers.fused_step import _FusedStep, _adamw_update, _sgd_update
from qtensor.utils import QTensorDiagReal

__all__ = ["CODE", "BlockPartitioner", "Preconditioner", "ShampooSGD", "ShampooAdamW"]


class Preconditioner(PreconditionerBase):
    """Compute statistics/shape from gradients for preconditioning (reference: shampoo1.py:102-244)."""

    def __init__(self, var, name2qmap, stat_decay=0.95, matrix_eps=1e-6, prec_maxorder=1200,
                 prec_bits=32, min_lowbit_size=4096, quan_blocksize=64):
        super().__init__(var, name2qmap, stat_decay=stat_decay, matrix_eps=matrix_eps, prec_maxorder=prec_maxorder,
                         prec_bits=prec_bits, min_lowbit_size=min_lowbit_size, quan_blocksize=quan_blocksize)

    def _new_statistic(self, order, device, index, rank, quant_args, extra):
        return QTensorDiagReal(self.matrix_eps * torch.eye(order, device=device), **quant_args)

    def _accumulate(self, holder, block, axis, w1, w2):
        # dequantize - decay - add Gram matrix - requantize (reference: shampoo1.py:164-179)
        if block.is_cuda and _fusable(holder):
            from qtensor import fused as X
            holder.quantize(X.gram(block, axis, stat=X.Quantized.from_holder(holder), beta=w1, alpha=w2))
            return
        stat = holder.dequantize()          # a dense holder hands out its own tensor: updated in place
        decay_and_add_gram(stat, block, axis, w1, w2)
        holder.quantize(stat)

    def _inverse_root(self, holder, exp, eps):
        # Like the reference (shampoo1.py:198), a statistic held in fp32 is passed without a copy,
        # so the ridge term the Newton routine adds in place stays in the stored statistic.
        stat = holder.dequantize()
        return newton_inverse_root(stat, exp, eps, getattr(self, '_v0', None)).to(stat.dtype)


class ShampooSGD(_FusedStep, ShampooSGDBase):
    __doc__ = _FusedStep.__doc__
    preconditioner_class = Preconditioner

    def __init__(self, params, *args, fused=False, **kwargs):
        super().__init__(params, *args, **kwargs)
        self._init_fused(fused)


class ShampooAdamW(_FusedStep, ShampooAdamWBase):
    __doc__ = _FusedStep.__doc__
    preconditioner_class = Preconditioner

    def __init__(self, params, *args, fused=False, **kwargs):
        super().__init__(params, *args, **kwargs)
        self._init_fused(fused)


ShampooSGD._update = staticmethod(_sgd_update)
ShampooAdamW._update = staticmethod(_adamw_update)
ShampooSGD.__doc__ = _DOC.format(base="SGD", more="") + _FusedStep.__doc__
ShampooAdamW.__doc__ = _DOC.format(base="AdamW", more="") + _FusedStep.__doc__
