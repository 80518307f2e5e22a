"""RMSNorm: ``y = x * 1/sqrt(mean(x^2) + eps) * w`` with eps inside the root
(kappai: src/backend/cpu/scalar/quants.c:1507-1512), computed in float32 and fused with the
residual sum that precedes it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from ..weights.spec import INIT_ONES, VECTOR, TensorSpec
from .base import Norm, register_part


class RMSNorm(Norm):
    can_defer = True      # add_norm(..., defer=True) may hand out an ops.PendingNorm

    def __init__(self, name: str, width: int, eps: float, dtype: torch.dtype):
        self.name, self.width, self.eps, self.dtype = name, width, float(eps), dtype
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + ".weight", (self.width,), VECTOR, INIT_ONES)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name + ".weight"].to(torch.float32).contiguous()

    def add_norm(self, resid, delta, rows=None, defer: bool = False):
        """``defer``: the caller's next part takes an ``ops.PendingNorm`` in place of the rows
        (a step with very few rows: the product kernel then makes them itself)."""
        if defer and rows is None and ops.PendingNorm.fits(resid, delta, self.dtype):
            return ops.PendingNorm(resid, delta, self.weight, self.eps, self.dtype)
        return ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.dtype, rows=rows,
                               write_resid=rows is None)

    def weight_bytes(self) -> int:
        return self.width * 4


register_part("norm", "rmsnorm", RMSNorm)
