"""Linear maps ``y = W x (+ b)`` with W stored [out, in] as in the checkpoint
(kappai: src/recipe/ops_basic.c:405, src/backend/cpu/scalar/quants.c:1398-1414)."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_NORMAL, INIT_SMALL, MATRIX, VECTOR, TensorSpec
from .base import Part


class Linear(Part):
    """One or several matrices of the checkpoint that share their input, run as ONE
    product: the matrices are stacked along their output dimension when they are bound
    (kappai's optional load-time fusion of q,k,v and gate,up, src/model.c:930-948)."""

    def __init__(self, names: Sequence[str], in_features: int, out_features: Sequence[int],
                 bias: bool = False, stage: str = "matmul", cut_rows_at: Sequence[int] = ()):
        """``cut_rows_at``: row counts at which the owner wants to use the first rows of the
        stacked matrix by themselves (``first_rows``)."""
        self.names = list(names)
        self.cut_rows_at = list(cut_rows_at)
        self.stage = stage              # the row of the --time table this product is booked under
        self.in_features = in_features
        self.out_features = list(out_features)
        self.has_bias = bias
        self.weight = None              # the matrix: a tensor [out, in], or ops.InFragments
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

    def bind(self, tensors: Dict[str, torch.Tensor], arrange=None) -> None:
        """``arrange(matrix) -> matrix``: another order of the stacked rows that the owner's
        kernel wants (gate and up rows interleaved), or None to keep them as they are."""
        ws = [tensors[n + ".weight"] for n in self.names]
        if len({w.dtype for w in ws}) > 1:           # stored in different widths: widen
            ws = [w.to(torch.float32) for w in ws]
        weight = ws[0] if len(ws) == 1 else torch.cat(ws, dim=0).contiguous()
        if arrange is not None:
            arranged = arrange(weight)
            weight = weight if arranged is None else arranged
        self.set_weight(weight)
        if self.has_bias:
            bs = [tensors[n + ".bias"].to(torch.float32) for n in self.names]
            self.bias = bs[0] if len(bs) == 1 else torch.cat(bs, dim=0).contiguous()

    def set_weight(self, weight: torch.Tensor) -> None:
        """The matrix of the product: kept in the order the product kernels load it when its
        shape allows that (and the rows that are used by themselves end on a piece), else as
        it is."""
        frag = None
        if tuning.FRAGMENT_ORDER and all(n % 16 == 0 for n in self.cut_rows_at):
            frag = ops.InFragments.of(weight)
        self.weight = weight if frag is None else frag

    def first_rows(self, n: int, stage: Optional[str] = None) -> "Linear":
        """A product with the first ``n`` rows of this one's matrix (and bias), sharing them."""
        if n not in self.cut_rows_at:
            raise ValueError(f"{self.names}: {n} is not among cut_rows_at {self.cut_rows_at}")
        part = Linear(self.names, self.in_features, [n], self.has_bias, stage or self.stage)
        w = self.weight
        part.weight = w.rows(n) if isinstance(w, ops.InFragments) else w[:n]
        part.bias = None if self.bias is None else self.bias[:n]
        return part

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
                              partial_sums=partial_sums, add_into=add_into)

    def weight_bytes(self) -> int:
        n = self.weight.numel() * self.weight.element_size()
        if self.bias is not None:
            n += self.bias.numel() * 4
        return n
