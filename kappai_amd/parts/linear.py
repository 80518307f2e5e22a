"""Linear maps ``y = W x (+ b)`` with W stored [out, in] as in the checkpoint
(kappai: src/recipe/ops_basic.c:405, src/backend/cpu/scalar/quants.c:1398-1414)."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_NORMAL, INIT_SMALL, MATRIX, VECTOR, TensorSpec
from .base import Part


# (how many rows, whether a second copy: kernels/tuning.py)


class Linear(Part):
    """One or several matrices of the checkpoint that share their input, run as ONE
    product: the matrices are stacked along their output dimension when they are bound
    (kappai's optional load-time fusion of q,k,v and gate,up, src/model.c:930-948)."""

    def __init__(self, names: Sequence[str], in_features: int, out_features: Sequence[int],
                 bias: bool = False, stage: str = "matmul"):
        self.names = list(names)
        self.stage = stage              # the row of the --time table this product is booked under
        self.in_features = in_features
        self.out_features = list(out_features)
        self.has_bias = bias
        self.weight: Optional[torch.Tensor] = None
        self.weight_frag: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    @property
    def total_out(self) -> int:
        return sum(self.out_features)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = []
        for n, o in zip(self.names, self.out_features):
            specs.append(TensorSpec(n + ".weight", (o, self.in_features), MATRIX, INIT_NORMAL))
            if self.has_bias:
                specs.append(TensorSpec(n + ".bias", (o,), VECTOR, INIT_SMALL))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        ws = [tensors[n + ".weight"] for n in self.names]
        if len({w.dtype for w in ws}) > 1:           # stored in different widths: widen
            ws = [w.to(torch.float32) for w in ws]
        self.set_weight(ws[0] if len(ws) == 1 else torch.cat(ws, dim=0).contiguous())
        if self.has_bias:
            bs = [tensors[n + ".bias"].to(torch.float32) for n in self.names]
            self.bias = bs[0] if len(bs) == 1 else torch.cat(bs, dim=0).contiguous()

    def set_weight(self, weight: torch.Tensor) -> None:
        """The matrix of the product, and its copy in fragment order when it is to have one."""
        self.weight = weight
        self.weight_frag = ops.fragment_order(weight) if tuning.FRAGMENT_COPIES else None

    def bind_shared(self, weight: torch.Tensor) -> None:
        """Use a tensor that another part owns (a tied output head)."""
        self.set_weight(weight)

    def forward(self, x: torch.Tensor, out_dtype=None, partial_sums: bool = False, add_into=None):
        """``partial_sums``: the caller hands the result to a norm as the pending residual
        update, which may then arrive as float32 sums over ranges of the input dimension.
        ``add_into`` (``ops.AddInto``): the product may add its result into the residual stream
        itself; what it returns then says so (``ops.Added``, ``ops.ScaledRows``)."""
        with profile.scope(self.stage, self.weight_bytes()):
            return ops.linear(x, self.weight, self.bias, out_dtype=out_dtype,
                              partial_sums=partial_sums, weight_frag=self.weight_frag,
                              add_into=add_into)

    def weight_bytes(self) -> int:
        n = self.weight.numel() * self.weight.element_size()
        if self.bias is not None:
            n += self.bias.numel() * 4
        return n
