"""Arrangements of parts in a layer."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..kernels import ops
from ..weights.spec import TensorSpec
from ctypes import Structure

from .base import Block, FeedForward, Hidden, Mixer, Norm, register_part, summed_delta
from .cdesc import NormPartDesc, PartDesc, defined_together


class PreNormBlockDesc(Structure):
    """``kappai_pre_norm_block`` of csrc/engine_parts.h."""
    _fields_ = [("mixer_norm", NormPartDesc), ("mixer", PartDesc), ("ffn_norm", NormPartDesc),
                ("feed_forward", PartDesc)]


def _takes_defer(norm) -> bool:
    return getattr(norm, "can_defer", False)


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

    @property
    def step_tables(self):
        return [t for t in (p.step_tables for p in self._parts()) if t is not None]

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self._parts() for s in p.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self._parts():
            p.bind(tensors)

    takes_next_block = True

    def first_norm(self):
        """The norm a block before this one may fold into its last product, and the part that
        takes its rows."""
        return self.mixer_norm, self.mixer

    def forward(self, h: Hidden, batch, cache, shared_cache: bool = False,
                next_block=None) -> Hidden:
        # decode steps with few rows: a product may add its result into the residual stream
        # itself and hand the next product its rows without a norm kernel in between
        resid = h.resid
        x = self._normed(self.mixer_norm, resid, h.delta, self.mixer)
        into = self._into(self.mixer, resid, self.ffn_norm, self.feed_forward)
        if into is not None:
            mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache, into=into)
        else:
            mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache)
        resid = self._resid_after(x, resid)
        x = self._normed(self.ffn_norm, resid, mixed, self.feed_forward)
        nxt = getattr(next_block, "first_norm", None)
        norm, consumer = nxt() if nxt is not None else (None, None)
        into = self._into(self.feed_forward, resid, norm, consumer)
        out = (self.feed_forward.forward(x, batch, into=into) if into is not None
               else self.feed_forward.forward(x, batch))
        return Hidden(self._resid_after(x, resid), out)

    @staticmethod
    def _into(producer, resid, norm, consumer):
        """What ``producer`` may add its result into, or None when it does not do such things."""
        if not getattr(producer, "adds_residual", False):
            return None
        fold = getattr(norm, "fold", None)
        if fold is not None and getattr(consumer, "takes_deferred_rows", False):
            return ops.AddInto(resid, *fold())
        return ops.AddInto(resid)

    @staticmethod
    def _normed(norm, resid, delta, consumer):
        delta = summed_delta(norm, delta)
        if getattr(consumer, "takes_deferred_rows", False) and _takes_defer(norm):
            return norm.add_norm(resid, delta, defer=True)
        return norm.add_norm(resid, delta)

    @staticmethod
    def _resid_after(x, resid):
        after = getattr(x, "resid_after", resid) if not isinstance(x, torch.Tensor) else resid
        if after is None:
            raise RuntimeError("a part that takes deferred rows did not use them")
        return after

    def c_call(self, plan, view, shared_cache: bool = False):
        """The block as the C side of a step runs it (runner "block.pre_norm"): the four parts'
        own descriptions side by side, or None when one of them has none.  A part whose class
        changed ``forward`` (or a norm's ``add_norm``) without giving a description of its own
        counts as having none."""
        for part, method, c_method in ((self.mixer_norm, "add_norm", "c_norm"),
                                       (self.mixer, "forward", "c_part"),
                                       (self.ffn_norm, "add_norm", "c_norm"),
                                       (self.feed_forward, "forward", "c_part")):
            if not defined_together(part, method, c_method):
                return None
        n1, n2 = self.mixer_norm.c_norm(plan), self.ffn_norm.c_norm(plan)
        mixer = self.mixer.c_part(plan, view, shared_cache)
        feed_forward = self.feed_forward.c_part(plan, None, False)
        if n1 is None or n2 is None or mixer is None or feed_forward is None:
            return None
        return plan.call("block.pre_norm", PreNormBlockDesc(n1, mixer, n2, feed_forward),
                         first_norm=n1, first_consumer=mixer)

    def weight_bytes(self) -> int:
        return sum(p.weight_bytes() for p in self._parts())


register_part("block", "pre_norm", PreNormBlock)
