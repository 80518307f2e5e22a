"""Arrangements of parts in a layer."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..weights.spec import TensorSpec
from .base import Block, FeedForward, Hidden, Mixer, Norm, register_part


class PreNormBlock(Block):
    """``x += mixer(norm(x)); x += feed_forward(norm(x))`` (kappai: src/models/lfm.c:7-53 with
    the tail src/recipe/builders.c:378-388).  Each residual sum is made inside the norm
    that follows it."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, feed_forward: FeedForward):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.ffn_norm, self.feed_forward = ffn_norm, feed_forward

    def _parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward)

    @property
    def capturable(self) -> bool:
        return all(p.capturable for p in self._parts())

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self._parts() for s in p.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self._parts():
            p.bind(tensors)

    def forward(self, h: Hidden, batch, cache, shared_cache: bool = False) -> Hidden:
        x = self.mixer_norm.add_norm(h.resid, h.delta)
        mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache)
        x = self.ffn_norm.add_norm(h.resid, mixed)
        return Hidden(h.resid, self.feed_forward.forward(x, batch))

    def weight_bytes(self) -> int:
        return sum(p.weight_bytes() for p in self._parts())


register_part("block", "pre_norm", PreNormBlock)
