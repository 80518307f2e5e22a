"""Token embedding and output head."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile
from ..weights.spec import INIT_NORMAL, TABLE, TensorSpec
from .base import Part
from .linear import Linear


class TokenEmbedding(Part):
    """Rows of the table widened to float32, without a scale
    (kappai: src/recipe/scratch.c:195-235)."""

    def __init__(self, name: str, vocab: int, width: int):
        self.name, self.vocab, self.width = name, vocab, width
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + ".weight", (self.vocab, self.width), TABLE, INIT_NORMAL)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name + ".weight"]

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        with profile.scope("embd"):
            return ops.embed_rows(tokens, self.table)

    def c_table(self):
        """The table as the C side of a step looks rows up in it."""
        return self.table

    def weight_bytes(self) -> int:
        return 0   # a step reads one row per token, not the table


class OutputHead(Part):
    """Logits in float32 for the rows asked for.  When tied the head is the embedding
    table itself (kappai: src/model.c:2562-2571)."""

    def __init__(self, name: str, vocab: int, width: int, tied_to: Optional[TokenEmbedding]):
        self.linear = Linear([name], width, [vocab], stage="logits_matmul")
        self.tied_to = tied_to

    def tensor_specs(self) -> List[TensorSpec]:
        return [] if self.tied_to is not None else self.linear.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        if self.tied_to is not None:
            self.linear.bind_shared(self.tied_to.table)
            if isinstance(self.linear.weight, ops.InFragments):
                # one matrix, in the order the products read it: the embedding reads that too
                self.tied_to.table = self.linear.weight
        else:
            self.linear.bind(tensors)

    takes_deferred_rows = True     # a plain product: it takes what ops.linear takes

    def forward(self, x) -> torch.Tensor:
        return self.linear.forward(x, out_dtype=torch.float32)

    def c_linear(self):
        """The head's product as the C side of a step runs it (float32 logits)."""
        return self.linear

    def weight_bytes(self) -> int:
        return self.linear.weight_bytes()
