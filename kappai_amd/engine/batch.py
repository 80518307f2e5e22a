"""The rows of one step and what the kernels need to know about them.

kappai describes a batch by a ``row_desc`` in one of three shapes: a portion of one
sequence, N single rows, or N segments (src/recipe.h:403-415, src/recipe/exec.c:925-981).
Here there is one shape: a list of segments, each a run of consecutive tokens of one
request; a decoded token is a segment of length one.
"""
from __future__ import annotations

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
    group g, logit_rows[n] (rows whose logits are wanted, in the order asked), q_tiles: the
    segments cut into runs of at most ``Model.q_tile_rows`` rows, laid out only when a part of
    the model asks for it (the tiled attention kernel does)."""
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
    q_tiles: Optional[torch.Tensor] = None      # [tiles, 4]: (segment, first row, rows, place)
    block_tables: List[torch.Tensor] = field(default_factory=list)
    host: Dict[str, np.ndarray] = field(default_factory=dict)


def tile_place(index: int, tiles_in_segment: int) -> int:
    """The fourth number of a q tile; 0 (place unknown) when the segment has more tiles than
    the 16 bits of either half hold."""
    if tiles_in_segment > 0x7fff:
        return 0
    return index | (tiles_in_segment << 16)


def layout_rows(entries: Sequence[StepEntry], cache: CacheManager, vocab_size: int,
                tile_rows: Optional[int] = None):
    """Host side of ``RowBatch``: checks the entries and lays the tables out as int32
    arrays.  Returns (dict of arrays, sizes).  ``tile_rows``: cut the segments into tiles of at
    most that many rows (``q_tiles``); None: no such table."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    seen = set()
    tokens, row_pos, row_seg, seg_start, seg_pos0, seg_slot, logit_rows = [], [], [], [0], [], [], []
    q_tiles = []
    max_position = 0
    for si, e in enumerate(entries):
        n = len(e.tokens)
        if n < 1:
            raise ValueError(f"entry {si} ({e.cache.request_id!r}) brings no tokens")
        if id(e.cache) in seen:
            raise ValueError(f"request {e.cache.request_id!r} appears twice in one step")
        seen.add(id(e.cache))
        toks = np.asarray(e.tokens, dtype=np.int64)
        if toks.ndim != 1 or int(toks.min()) < 0 or int(toks.max()) >= vocab_size:
            bad = next(int(t) for t in toks.reshape(-1) if not 0 <= int(t) < vocab_size)
            raise ValueError(f"entry {si} ({e.cache.request_id!r}): token id {bad} is outside "
                             f"the vocabulary of {vocab_size}")
        for w in e.want:
            if not 0 <= int(w) < n:
                raise ValueError(f"entry {si} ({e.cache.request_id!r}): wanted place {w} is "
                                 f"outside its {n} tokens")
        base = seg_start[-1]
        p0 = e.cache.length
        tokens.append(toks.astype(np.int32))
        row_pos.append(np.arange(p0, p0 + n, dtype=np.int32))
        row_seg.append(np.full(n, si, dtype=np.int32))
        max_position = max(max_position, p0 + n - 1)
        seg_start.append(base + n)
        if tile_rows:
            n_seg_tiles = (n + tile_rows - 1) // tile_rows
            for j, r in enumerate(range(0, n, tile_rows)):
                # the fourth number tells a kernel where the tile stands in its segment
                # (index | tiles of the segment << 16), so that it can pair tiles of one segment
                q_tiles.append((si, base + r, min(tile_rows, n - r), tile_place(j, n_seg_tiles)))
        seg_pos0.append(p0)
        seg_slot.append(e.cache.slot)
        logit_rows.extend(base + int(w) for w in e.want)
    S = len(entries)
    tables = []
    for gi in range(len(cache.paged_groups)):
        width = max(1, max(len(e.cache.blocks[gi]) for e in entries))
        bt = np.full((S, width), -1, dtype=np.int32)
        for si, e in enumerate(entries):
            b = e.cache.blocks[gi]
            bt[si, :len(b)] = b
        tables.append(bt)
    arrays = {
        "tokens": np.concatenate(tokens),
        "row_pos": np.concatenate(row_pos),
        "row_seg": np.concatenate(row_seg),
        "seg_start": np.asarray(seg_start, dtype=np.int32),
        "seg_pos0": np.asarray(seg_pos0, dtype=np.int32),
        "seg_slot": np.asarray(seg_slot, dtype=np.int32),
        "logit_rows": np.asarray(logit_rows, dtype=np.int32),
    }
    if tile_rows:
        arrays["q_tiles"] = np.asarray(q_tiles, dtype=np.int32).reshape(-1, 4)
    for gi, bt in enumerate(tables):
        arrays[f"block_table_{gi}"] = bt
    sizes = {
        "n_rows": seg_start[-1], "n_segments": S, "n_logit_rows": len(logit_rows),
        "max_position": max_position,
        "max_segment_rows": max(len(e.tokens) for e in entries),
        "n_groups": len(tables),
    }
    return arrays, sizes
