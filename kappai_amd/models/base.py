"""A model as data: blocks, and the order in which they run.

``schedule`` is a list of ``LayerCall``: which block runs, and which cache it uses.  A
block may be named more than once (then every call has a cache of its own), and a call
may read the cache that an earlier call wrote instead of owning one (``reads_cache_of``).
The caches are numbered by the calls that own them; the cache manager groups them by
what they need.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from ..config.base import ModelConfig
from ..kernels import ops
from ..parts.base import Block, Hidden, Norm, PositionEncoding, summed_delta
from ..parts.embedding import OutputHead, TokenEmbedding
from ..weights.spec import TensorSpec


@dataclass(frozen=True)
class LayerCall:
    layer: int                            # index into Model.layers
    reads_cache_of: Optional[int] = None  # index into the schedule of the call whose cache is read


class Model:
    def __init__(self, config: ModelConfig, dtype: torch.dtype, embedding: TokenEmbedding,
                 layers: Sequence[Block], final_norm: Norm, head: OutputHead,
                 schedule: Optional[Sequence[LayerCall]] = None,
                 embedding_position: Optional[PositionEncoding] = None):
        self.config, self.dtype = config, dtype
        self.embedding, self.layers = embedding, list(layers)
        self.final_norm, self.head = final_norm, head
        self.embedding_position = embedding_position
        self.schedule: List[LayerCall] = list(schedule) if schedule is not None else [
            LayerCall(i) for i in range(len(self.layers))]
        self._check_schedule()
        self.bound = False

    def _check_schedule(self) -> None:
        for ci, call in enumerate(self.schedule):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"schedule[{ci}] names layer {call.layer}; there are "
                                 f"{len(self.layers)}")
            src = call.reads_cache_of
            if src is not None:
                if not 0 <= src < ci:
                    raise ValueError(f"schedule[{ci}] reads the cache of call {src}, which does "
                                     f"not run before it")
                if self.schedule[src].reads_cache_of is not None:
                    raise ValueError(f"schedule[{ci}] reads the cache of call {src}, which owns none")
                a = self.layers[call.layer].cache_spec()
                b = self.layers[self.schedule[src].layer].cache_spec()
                if a != b:
                    raise ValueError(f"schedule[{ci}] needs {a} but call {src} keeps {b}")

    # -- caches ----------------------------------------------------------------------------
    def cache_specs(self) -> list:
        """One entry per call of the schedule: what its own cache needs, or None when the
        call owns none."""
        return [None if c.reads_cache_of is not None else self.layers[c.layer].cache_spec()
                for c in self.schedule]

    def cache_id(self, call_index: int) -> int:
        c = self.schedule[call_index]
        return call_index if c.reads_cache_of is None else c.reads_cache_of

    # -- weights ---------------------------------------------------------------------------
    def _parts(self):
        parts = [self.embedding, *self.layers, self.final_norm, self.head]
        if self.embedding_position is not None:
            parts.append(self.embedding_position)
        return parts

    def tensor_specs(self) -> List[TensorSpec]:
        seen: Dict[str, TensorSpec] = {}
        for p in self._parts():
            for s in p.tensor_specs():
                if s.name in seen and seen[s.name] != s:
                    raise ValueError(f"tensor {s.name} is declared twice with different shapes")
                seen[s.name] = s
        return list(seen.values())

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self._parts():
            p.bind(tensors)
        self.bound = True

    def weight_bytes_per_step(self) -> int:
        """Bytes of weights a step reads once: every block as often as the schedule runs it,
        the final norm and the head."""
        n = sum(self.layers[c.layer].weight_bytes() for c in self.schedule)
        return n + self.final_norm.weight_bytes() + self.head.weight_bytes()

    @property
    def capturable(self) -> bool:
        """True if every part allows decode steps to be captured in HIP graphs."""
        return all(getattr(p, "capturable", True) for p in self._parts())

    def step_tables(self) -> list:
        """The tables that the parts ask of a step beside the framework's own
        (``parts.base.StepTables``), one set per family."""
        families = {}
        for part in [*self.layers, self.embedding_position]:
            asked = getattr(part, "step_tables", None)
            if asked is None:
                continue
            for t in (asked if isinstance(asked, (list, tuple)) else [asked]):
                families.setdefault(t.family, []).append(t)
        return [ts[0].combine(ts[1:]) for ts in families.values()]

    @property
    def vocab_size(self) -> int:
        return self.config.vocab_size

    def first_norm(self):
        """What the last block of the schedule sees in place of a next block: the final norm and
        the head that takes its rows."""
        return self.final_norm, self.head

    def c_calls(self, plan):
        """The schedule as the C side of a step runs it: every call's block described by itself
        (``Block.c_call``), or None when a block has no description.  The C walk does what
        ``forward`` below does, which is why the two are defined side by side: a subclass that
        changes ``forward`` gets no walk from C unless it describes one."""
        from ..parts.cdesc import defined_together
        calls = []
        for ci, call in enumerate(self.schedule):
            block = self.layers[call.layer]
            if not defined_together(block, "forward", "c_call"):
                return None
            view = plan.cache.view(self.cache_id(ci)) if block.cache_spec() is not None else None
            described = block.c_call(plan, view, call.reads_cache_of is not None)
            if described is None:
                return None
            calls.append(described)
        return calls

    # -- the forward pass of one step ------------------------------------------------------
    def forward(self, batch, cache) -> torch.Tensor:
        """Run the rows of ``batch`` through every call of the schedule and return float32
        logits [len(batch.logit_rows), vocab] (kappai: compute_forward_rows,
        src/recipe/exec.c:704-758)."""
        if not self.bound:
            raise RuntimeError("the model has no weights yet: call bind() or load_model()")
        x = self.embedding.forward(batch.tokens)
        if self.embedding_position is not None:
            self.embedding_position.on_embedding(x, batch)
        h = Hidden(x, None)
        for ci, call in enumerate(self.schedule):
            block = self.layers[call.layer]
            view = None
            if block.cache_spec() is not None:
                view = cache.view(self.cache_id(ci))
            shared = call.reads_cache_of is not None
            if getattr(block, "takes_next_block", False):
                if ci + 1 < len(self.schedule):
                    nxt = self.layers[self.schedule[ci + 1].layer]
                else:
                    # after the last call comes the final norm, whose rows the head takes; a
                    # block can make them only when every row wants its logits
                    nxt = self if getattr(batch, "logits_of_every_row", False) else None
                h = block.forward(h, batch, view, shared_cache=shared, next_block=nxt)
            else:
                h = block.forward(h, batch, view, shared_cache=shared)
        if batch.n_logit_rows == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=x.device)
        delta = summed_delta(self.final_norm, h.delta)
        if (getattr(self.final_norm, "can_defer", False)
                and getattr(self.head, "takes_deferred_rows", False)):
            made = (isinstance(delta, ops.ScaledRows)
                    and getattr(batch, "logits_of_every_row", False))
            xb = self.final_norm.add_norm(h.resid, delta, rows=None if made else batch.logit_rows,
                                          defer=True)
        else:
            xb = self.final_norm.add_norm(h.resid, delta, rows=batch.logit_rows)
        return self.head.forward(xb)
