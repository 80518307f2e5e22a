"""SwiGLU feed-forward: ``W2 (silu(W1 x) * W3 x)`` (kappai: src/recipe/builders.c:344-370,
383-386; silu at src/backend/cpu/quants.h:369-371).  W1 and W3 are stacked into one
product."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import FeedForward, register_part
from .linear import Linear


class SwiGLU(FeedForward):
    def __init__(self, prefix: str, width: int, hidden: int, dtype: torch.dtype, names=None):
        n = {"gate": "w1", "up": "w3", "down": "w2"}
        n.update(names or {})
        self.width, self.hidden, self.dtype = width, hidden, dtype
        self.gate_up = Linear([prefix + n["gate"], prefix + n["up"]], width, [hidden, hidden])
        self.down = Linear([prefix + n["down"]], hidden, [width])

    def tensor_specs(self) -> List[TensorSpec]:
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gate_up.bind(tensors)
        self.down.bind(tensors)

    def forward(self, x, batch):
        return self.down.forward(ops.swiglu(self.gate_up.forward(x)))

    def weight_bytes(self) -> int:
        return self.gate_up.weight_bytes() + self.down.weight_bytes()


register_part("feed_forward", "swiglu", SwiGLU)
