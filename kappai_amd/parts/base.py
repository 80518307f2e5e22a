"""The interfaces that layers are put together from, and the registries that a
configuration chooses parts by.

A model is a list of blocks and a list that says in which order they run.  A block
arranges a norm, a token mixer, a second norm and a feed-forward; each of those is a
part with its sizes and constants as constructor arguments.  No part knows which model
it is in: it sees its own tensors, the rows of the step (``RowBatch``) and, if it asked
for one, its view of the cache.

Adding a part means writing a class with the interface below and registering it under a
name; an architecture's builder then picks it layer by layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional

import torch

from ..weights.spec import TensorSpec


class StepTables:
    """More int32 tables of a step, laid out on the host for a part whose kernels want them (the
    segments cut into tiles, some rows listed apart, the chunks of a scan, ...).

    ``family``: tables of one family are built once a step, however many layers ask for them;
    ``combine`` says what is built when the layers ask differently.  ``build(step)`` gets the
    step's own tables on the host (``step.arrays``: tokens, row_pos, row_seg, seg_start,
    seg_pos0, seg_slot, logit_rows as numpy int32 arrays; ``step.sizes``: n_rows, n_segments,
    max_position, max_segment_rows; ``step.page_size``) and returns ``(arrays, numbers)``: more
    int32 arrays by name, and ints by name that stay on the host (what a launch is sized by).
    Names are the family's own; an array that is not needed in a step is left out.
    ``decode_constant``: in a step of nothing but single rows the arrays depend on the number of
    rows only, so that a captured decode graph fills them in once; else they are built again for
    every replay and must keep their shapes."""

    family: str = ""
    decode_constant: bool = False

    def build(self, step):
        raise NotImplementedError

    def combine(self, others: List["StepTables"]) -> "StepTables":
        """The one set of tables for ``self`` and ``others`` of the same family."""
        for o in others:
            if o != self:
                raise ValueError(f"layers ask for different tables of the family {self.family!r}: "
                                 f"{self!r} and {o!r}")
        return self


class Part:
    """Anything that owns tensors of the checkpoint."""

    # True if ``forward`` only launches GPU work whose shapes depend on the batch's sizes, not
    # on its contents, so that a decode step may be captured in a HIP graph and replayed.  A
    # part that reads the batch's tables on the host sets this to False.
    capturable = True

    # More tables of the step that the part's kernels want beside the framework's own (a
    # ``StepTables``), or None.  The step function builds them on the host with its own tables and
    # brings them to the GPU in the same copy: ``RowBatch.extra[name]``, ``RowBatch.numbers[name]``.
    step_tables: Optional["StepTables"] = None

    def tensor_specs(self) -> List[TensorSpec]:
        """Full names, shapes and roles of the tensors this part reads from the file."""
        return []

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Take the loaded tensors (by full name) and lay them out for the kernels."""

    def weight_bytes(self) -> int:
        """Bytes of weights that one step reads from this part."""
        return 0


class Norm(Part):
    """``add_norm`` adds ``delta`` (may be None) into the float32 residual in place and
    returns the normalised rows in the compute dtype.  With ``rows`` only those rows are
    normalised and the residual is left as it is.

    ``delta`` is [T, width] in the compute dtype or in float32.  The parts before a norm may
    also hand on float32 partial sums [S, T, width] of a product split over its input
    dimension; a norm that adds them itself (in order, in float32) says so with
    ``takes_partial_sums = True``, any other norm gets them summed by ``summed_delta`` (what
    blocks and the model call before ``add_norm``) and never sees three dimensions."""

    takes_partial_sums = False

    def add_norm(self, resid: torch.Tensor, delta: Optional[torch.Tensor],
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


def summed_delta(norm: Norm, delta):
    """``delta`` as ``norm`` takes it: partial sums [S, T, width] are added up first unless the
    norm adds them itself, and what a product returns that has added its result into the
    residual itself (``ops.Added``) becomes None unless the norm knows of such things."""
    from ..kernels import ops
    if isinstance(delta, ops.Added) and not getattr(norm, "can_defer", False):
        return None                  # a product has added its result into the residual itself
    if (isinstance(delta, torch.Tensor) and delta.dim() == 3
            and not getattr(norm, "takes_partial_sums", False)):
        return ops.sum_partial_sums(delta)
    return delta


class PositionEncoding(Part):
    """How positions enter the model.  ``rotation(max_position)`` gives what the attention
    kernels rotate queries and keys with (or None); ``on_embedding`` may change the
    embedded rows in place (absolute encodings)."""

    def rotation(self, device, max_position: int):
        return None

    def on_embedding(self, x: torch.Tensor, batch) -> None:
        return None


class Mixer(Part):
    """A token mixer.  ``cache_spec`` says what it needs from the cache manager (a PagedSpec,
    FixedState or None); ``forward`` gets the normalised rows [T, width] in the compute
    dtype, the step's ``RowBatch`` and its cache view, and returns [T, width] in the compute
    dtype, or float32 partial sums [S, T, width] that the next norm adds up.

    Two optional abilities, for decode steps with few rows, each announced by a flag:
    ``takes_deferred_rows = True``: ``x`` may arrive as ``ops.ScaledRows`` or
    ``ops.FragmentRows`` (what ``ops.linear`` and its relatives take in place of rows) when the
    norm before the part can hand them out.
    ``adds_residual = True``: ``forward`` takes ``into=ops.AddInto(...)`` (or None) and passes it
    to its last product, which then adds the result into the residual stream itself and folds
    the following norm in; the part returns what that product returned."""

    takes_deferred_rows = False
    adds_residual = False

    def cache_spec(self):
        return None

    def forward(self, x: torch.Tensor, batch, cache, shared_cache: bool = False) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """``forward(x, batch)`` returns [T, width] or float32 partial sums [S, T, width].  The two
    optional abilities of ``Mixer`` (``takes_deferred_rows``, ``adds_residual`` with an ``into``
    argument) hold here as well."""

    takes_deferred_rows = False
    adds_residual = False

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


@dataclass
class Hidden:
    """The residual stream between blocks: ``resid`` (float32, [T, width]) and the last
    part's output ``delta`` that has not been added yet ([T, width], or float32 partial sums
    [S, T, width]).  The next norm adds it while it normalises, so the sum is made in float32
    and costs no pass of its own."""
    resid: torch.Tensor
    delta: Optional[object] = None      # a tensor, or ops.Added / ops.ScaledRows: nothing to add


class Block(Part):
    """An arrangement of parts around the residual stream."""

    mixer: Mixer

    # True if ``forward`` takes ``next_block``: the block that runs after this one (None after
    # the last), so that this block's last product can fold that block's first norm in.
    takes_next_block = False

    def cache_spec(self):
        return self.mixer.cache_spec()

    @property
    def step_tables(self):
        """The tables its parts ask of a step (a list)."""
        asked = getattr(self.mixer, "step_tables", None)
        return [] if asked is None else [asked]

    def forward(self, h: Hidden, batch, cache, shared_cache: bool = False) -> Hidden:
        raise NotImplementedError


# --------------------------------------------------------------------------------------
# registries: name -> constructor
# --------------------------------------------------------------------------------------
MIXERS: Dict[str, Callable[..., Mixer]] = {}
FEED_FORWARDS: Dict[str, Callable[..., FeedForward]] = {}
NORMS: Dict[str, Callable[..., Norm]] = {}
POSITION_ENCODINGS: Dict[str, Callable[..., PositionEncoding]] = {}
BLOCKS: Dict[str, Callable[..., Block]] = {}

_REGISTRIES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS,
               "position_encoding": POSITION_ENCODINGS, "block": BLOCKS}


def register_part(kind: str, part_name: str, ctor: Callable) -> None:
    if kind not in _REGISTRIES:
        raise KeyError(f"unknown kind of part {kind!r}; known: {', '.join(_REGISTRIES)}")
    _REGISTRIES[kind][part_name] = ctor


def make_part(kind: str, part_name: str, /, **kwargs):
    """Construct the part registered as ``part_name``; ``kwargs`` go to its constructor."""
    if kind not in _REGISTRIES:
        raise KeyError(f"unknown kind of part {kind!r}; known: {', '.join(_REGISTRIES)}")
    reg = _REGISTRIES[kind]
    if part_name not in reg:
        raise KeyError(f"no {kind} named {part_name!r}; known: {', '.join(sorted(reg)) or 'none'}")
    return reg[part_name](**kwargs)
