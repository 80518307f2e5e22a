"""RMSNorm: ``y = x * 1/sqrt(mean(x^2) + eps) * w`` with eps inside the root
(kappai: src/backend/cpu/scalar/quants.c:1507-1512), computed in float32 and fused with the
residual sum that precedes it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_ONES, VECTOR, TensorSpec
from .base import Norm, register_part
from .cdesc import FoldDesc


class RMSNorm(Norm):
    takes_partial_sums = True      # the kernel adds [S, T, width] partial sums itself, in order
    can_defer = True      # add_norm(..., defer=True) may hand out ops.ScaledRows or
                          # ops.FragmentRows in place of a tensor

    def __init__(self, name: str, width: int, eps: float, dtype: torch.dtype):
        self.name, self.width, self.eps, self.dtype = name, width, float(eps), dtype
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + ".weight", (self.width,), VECTOR, INIT_ONES)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name + ".weight"].to(torch.float32).contiguous()

    def fold(self):
        """(weight, eps) for a product that folds this norm in (``ops.AddInto``): the norm is
        ``x * weight / rms(x)``, so the product before it can hand on ``x * weight`` and the sums
        of squares, and the product after it divides."""
        return self.weight, self.eps

    def add_norm(self, resid, delta, rows=None, defer: bool = False):
        """``delta`` may also be what a product hands back that has added its result into
        ``resid`` itself: ``ops.Added``, or ``ops.ScaledRows`` made for this norm.  ``defer``: the
        caller's next part takes what the product kernels take in place of the rows: such
        ``ops.ScaledRows`` as they are, or ``ops.FragmentRows`` (8 to 16 rows, made here in the
        order the product loads them)."""
        if isinstance(delta, ops.Added):
            if (defer and rows is None and isinstance(delta, ops.ScaledRows)
                    and delta.weight is self.weight and delta.eps == self.eps
                    and delta.resid is resid):
                return delta
            delta = None             # the sum is in ``resid`` already
        n = resid.shape[0] if rows is None else rows.shape[0]
        fragment = (defer and tuning.FRAGMENT_ROWS and resid.is_cuda
                    and n >= tuning.FRAGMENT_ROWS_MIN
                    and ops.FragmentRows.fits(n, self.width, self.dtype)
                    and (delta is None or delta.dim() == 2 or delta.shape[0] <= 8))
        with profile.scope("rmsnorm" if rows is None else "logits_norm"):
            return ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.dtype, rows=rows,
                                   write_resid=rows is None, fragment=fragment)

    def c_norm(self, plan):
        """The norm as the C side of a step runs it: the runner "norm.rms" reads weight and eps,
        which is also all a product needs to fold the norm in."""
        fold = plan.keep(FoldDesc(self.weight.data_ptr(), self.eps))
        return plan.norm("norm.rms", fold, fold=fold)

    def weight_bytes(self) -> int:
        return self.width * 4


register_part("norm", "rmsnorm", RMSNorm)
