"""The rows of one step and what the kernels need to know about them.

kappai describes a batch by a ``row_desc`` in one of three shapes: a portion of one
sequence, N single rows, or N segments (src/recipe.h:403-415, src/recipe/exec.c:925-981).
Here there is one shape: a list of segments, each a run of consecutive tokens of one
request; a decoded token is a segment of length one.
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, RequestCache


@dataclass
class StepEntry:
    """One request's part of a step: its next ``tokens`` (they follow what its cache holds)
    and ``want``, the places among these tokens whose logits are asked for."""
    cache: RequestCache
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class RowBatch:
    """Device tables of a step.  T rows, S segments.

    tokens[T], row_pos[T] (absolute position), row_seg[T] (segment of the row),
    seg_start[S+1] (first row of each segment), seg_pos0[S] (position of that row),
    seg_slot[S] (the request's state slot), block_tables[g] [S, max_blocks] for every paged
    group g, logit_rows[n] (rows whose logits are wanted, in the order asked;
    ``logits_of_every_row``: these are the rows 0 .. T-1 in order, which the host knows and a
    part that could fold the last norm into a product cannot read from the GPU).  ``extra`` and
    ``numbers``: what the parts' own ``StepTables`` laid out for this step, tables on the GPU and
    ints on the host, by name."""
    n_rows: int
    n_segments: int
    n_logit_rows: int
    max_position: int
    max_segment_rows: int
    tokens: torch.Tensor
    row_pos: torch.Tensor
    row_seg: torch.Tensor
    seg_start: torch.Tensor
    seg_pos0: torch.Tensor
    seg_slot: torch.Tensor
    logit_rows: torch.Tensor
    extra: Dict[str, torch.Tensor] = field(default_factory=dict)
    numbers: Dict[str, int] = field(default_factory=dict)
    logits_of_every_row: bool = False
    block_tables: List[torch.Tensor] = field(default_factory=list)
    host: Dict[str, np.ndarray] = field(default_factory=dict)


@dataclass
class HostStep:
    """What a ``StepTables`` builds from: the step's own tables on the host."""
    arrays: Dict[str, np.ndarray]
    sizes: Dict[str, object]
    page_size: int


def build_step_tables(tables, step: HostStep):
    """Every family's arrays and numbers for this step: ({name: int32 array}, {name: int})."""
    arrays: Dict[str, np.ndarray] = {}
    numbers: Dict[str, int] = {}
    for t in tables:
        made, nums = t.build(step)
        for name, a in made.items():
            if name in arrays or name in step.arrays:
                raise ValueError(f"two tables of a step are called {name!r}")
            if a.dtype != np.int32:
                raise ValueError(f"the table {name!r} of {t.family!r} is not int32")
            arrays[name] = a
        for name, v in nums.items():
            if name in numbers:
                raise ValueError(f"two numbers of a step are called {name!r}")
            numbers[name] = int(v)
    return arrays, numbers


def tile_place(index: int, tiles_in_segment: int) -> int:
    """The fourth number of a q tile; 0 (place unknown) when the segment has more tiles than
    the 16 bits of either half hold."""
    if tiles_in_segment > 0x7fff:
        return 0
    return index | (tiles_in_segment << 16)


def layout_rows(entries: Sequence[StepEntry], cache: CacheManager, vocab_size: int, tables=()):
    """Host side of ``RowBatch``: checks the entries and lays the tables out as int32
    arrays.  Returns (dict of arrays, sizes).  ``tables``: the ``StepTables`` of the model's
    parts, whose arrays join the dict (their names in ``sizes["extra"]``, their numbers in
    ``sizes["numbers"]``).  The tables are made for all entries at once (a step of many single
    decoded tokens costs a few numpy calls, not a few per entry)."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    S = len(entries)
    seen = set()
    counts, pos0, slots, logit_rows = [], [], [], []
    base = 0
    for si, e in enumerate(entries):
        n = len(e.tokens)
        if n < 1:
            raise ValueError(f"entry {si} ({e.cache.request_id!r}) brings no tokens")
        if id(e.cache) in seen:
            raise ValueError(f"request {e.cache.request_id!r} appears twice in one step")
        seen.add(id(e.cache))
        for w in e.want:
            if not 0 <= int(w) < n:
                raise ValueError(f"entry {si} ({e.cache.request_id!r}): wanted place {w} is "
                                 f"outside its {n} tokens")
            logit_rows.append(base + int(w))
        counts.append(n)
        pos0.append(e.cache.length)
        slots.append(e.cache.slot)
        base += n
    T = base
    try:
        tokens = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries),
                             dtype=np.int64, count=T)
    except (TypeError, ValueError):
        tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int64).reshape(-1)
                                 for e in entries])
    if int(tokens.min()) < 0 or int(tokens.max()) >= vocab_size:
        at = int(np.flatnonzero((tokens < 0) | (tokens >= vocab_size))[0])
        si = int(np.searchsorted(np.cumsum(counts), at, side="right"))
        raise ValueError(f"entry {si} ({entries[si].cache.request_id!r}): token id "
                         f"{int(tokens[at])} is outside the vocabulary of {vocab_size}")
    n_arr = np.asarray(counts, dtype=np.int64)
    p0_arr = np.asarray(pos0, dtype=np.int64)
    seg_start = np.zeros(S + 1, dtype=np.int64)
    np.cumsum(n_arr, out=seg_start[1:])
    row_seg = np.repeat(np.arange(S, dtype=np.int64), n_arr)
    row_pos = np.arange(T, dtype=np.int64) - np.repeat(seg_start[:-1] - p0_arr, n_arr)
    max_position = int((p0_arr + n_arr).max()) - 1
    arrays = {
        "tokens": tokens.astype(np.int32),
        "row_pos": row_pos.astype(np.int32),
        "row_seg": row_seg.astype(np.int32),
        "seg_start": seg_start.astype(np.int32),
        "seg_pos0": p0_arr.astype(np.int32),
        "seg_slot": np.asarray(slots, dtype=np.int32),
        "logit_rows": np.asarray(logit_rows, dtype=np.int32),
    }
    n_groups = len(cache.paged_groups)
    for gi in range(n_groups):
        width = max(1, max(len(e.cache.blocks[gi]) for e in entries))
        bt = np.full((S, width), -1, dtype=np.int32)
        for si, e in enumerate(entries):
            b = e.cache.block_array(gi)      # (kept by the request until its pages change)
            bt[si, :b.size] = b
        arrays[f"block_table_{gi}"] = bt
    sizes = {
        "n_rows": T, "n_segments": S, "n_logit_rows": len(logit_rows),
        "max_position": max_position, "max_segment_rows": int(n_arr.max()),
        "n_groups": n_groups,
        "logits_of_every_row": logit_rows == list(range(T)),
    }
    extra, numbers = build_step_tables(tables, HostStep(arrays, sizes, cache.page_size))
    arrays.update(extra)
    sizes["extra"] = list(extra)
    sizes["numbers"] = numbers
    return arrays, sizes
