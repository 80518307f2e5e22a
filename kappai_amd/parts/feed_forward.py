"""SwiGLU feed-forward: ``W2 (silu(W1 x) * W3 x)`` (kappai: src/recipe/builders.c:344-370,
383-386; silu at src/backend/cpu/quants.h:369-371).  W1 and W3 are stacked into one
product; in bfloat16 their rows are interleaved so that the product's epilogue applies the
gate and the [T, 2F] intermediate never reaches memory."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..kernels import ops, profile
from ..weights.spec import TensorSpec
from ctypes import Structure, c_int

from .base import FeedForward, register_part
from .cdesc import LinearDesc
from .linear import Linear


class SwiGLUDesc(Structure):
    """``kappai_swiglu`` of csrc/engine_parts.h."""
    _fields_ = [("gate_up", LinearDesc), ("down", LinearDesc), ("hidden", c_int),
                ("fused", c_int)]


class SwiGLU(FeedForward):
    takes_deferred_rows = True     # its first product takes what ops.linear takes
    adds_residual = True           # its last product can add into the residual stream

    def __init__(self, prefix: str, width: int, hidden: int, dtype: torch.dtype, names=None):
        n = {"gate": "w1", "up": "w3", "down": "w2"}
        n.update(names or {})
        self.width, self.hidden, self.dtype = width, hidden, dtype
        self.fused = False
        self.gate_up = Linear([prefix + n["gate"], prefix + n["up"]], width, [hidden, hidden],
                              stage="matmul_ffn_gate_up")
        self.down = Linear([prefix + n["down"]], hidden, [width], stage="matmul_ffn_down")

    def tensor_specs(self) -> List[TensorSpec]:
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        def interleaved(w):
            # the fused product wants gate and up rows in turns of 16
            self.fused = (w.dtype == torch.bfloat16 and self.hidden % ops.SWIGLU_GROUP == 0
                          and self.width % 8 == 0)
            return ops.interleave_gate_up(w[:self.hidden], w[self.hidden:]) if self.fused else None

        self.gate_up.bind(tensors, arrange=interleaved)
        self.down.bind(tensors)

    def forward(self, x, batch, into=None):
        if self.fused and x.dtype == torch.bfloat16:
            with profile.scope("matmul_ffn_gate_up", self.gate_up.weight_bytes()):
                act = ops.linear_swiglu(x, self.gate_up.weight, out_fragment=True)
            return self.down.forward(act, partial_sums=True, add_into=into)
        gate_up = self.gate_up.forward(x)
        with profile.scope("ffn_act"):
            act = ops.swiglu(gate_up)
        return self.down.forward(act, partial_sums=True, add_into=into)

    def c_part(self, plan, view=None, shared_cache: bool = False):
        """The runner "feed_forward.swiglu" (csrc/engine_parts.hip) makes the same choices as
        ``forward``."""
        first = plan.linear(self.gate_up)
        desc = SwiGLUDesc(first, plan.linear(self.down), self.hidden, 1 if self.fused else 0)
        return plan.part("feed_forward.swiglu", desc, takes_deferred_rows=True,
                         adds_residual=True, first=first)

    def weight_bytes(self) -> int:
        return self.gate_up.weight_bytes() + self.down.weight_bytes()


register_part("feed_forward", "swiglu", SwiGLU)
