"""The step function: a batch of (request, its next tokens) in, logits at the wanted
places out.

kappai has four step functions over one executor (compute_forward, compute_forward_batch,
compute_forward_decode_batch, compute_forward_segments; src/compute.c:271-380,
src/compute.h:120-149) and never mixes prompt portions with decoded tokens.  Here one
function takes any mixture: it makes room in the cache for the new tokens, lays out the
row tables, copies them to the GPU in one transfer, runs the model over exactly these
rows and commits the new lengths.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, OutOfPages
from ..models.base import Model
from .batch import RowBatch, StepEntry, layout_rows


CONTEXT_BUCKET_MIN = 1024     # decode graphs are captured for contexts up to a power of two
MAX_DECODE_GRAPHS = 48


def _context_bucket(n_positions: int) -> int:
    cap = CONTEXT_BUCKET_MIN
    while cap < n_positions:
        cap *= 2
    return cap


class _DecodeGraph:
    """One captured HIP graph of the model's forward pass for B single-token segments whose
    positions lie below ``ctx_cap``: static row tables that every step overwrites, a static
    logits tensor that every replay fills."""

    def __init__(self, runner: "StepRunner", arrays, sizes, ctx_cap: int):
        self.order = list(arrays)
        self.shapes = {k: arrays[k].shape for k in self.order}
        self.offsets, total = {}, 0
        for k in self.order:
            self.offsets[k] = total
            total += (arrays[k].size + 3) // 4 * 4
        self.total = max(total, 4)
        dev = runner.device
        self.static = torch.zeros(self.total, dtype=torch.int32, device=dev)
        views = {k: self.static[self.offsets[k]:self.offsets[k] + arrays[k].size].view(
            arrays[k].shape) for k in self.order}
        B = sizes["n_rows"]
        self.batch = RowBatch(
            n_rows=B, n_segments=B, n_logit_rows=sizes["n_logit_rows"], max_position=ctx_cap - 1,
            max_segment_rows=1, tokens=views["tokens"], row_pos=views["row_pos"],
            row_seg=views["row_seg"], seg_start=views["seg_start"], seg_pos0=views["seg_pos0"],
            seg_slot=views["seg_slot"], logit_rows=views["logit_rows"], q_tiles=views["q_tiles"],
            block_tables=[views[f"block_table_{g}"] for g in range(sizes["n_groups"])], host={})
        # a warm-up run on the scratch page and the scratch slot: every kernel of this shape is
        # loaded and has run once before the capture, and no request's cache is touched
        cache = runner.cache
        warm = {k: np.zeros(arrays[k].shape, dtype=np.int32) for k in self.order}
        warm["row_seg"][:] = np.arange(B)
        warm["seg_start"][:] = np.arange(B + 1)
        warm["seg_slot"][:] = cache.scratch_slot
        warm["logit_rows"][:] = np.arange(sizes["n_logit_rows"]) % B
        warm["q_tiles"][:, 0] = np.arange(B)
        warm["q_tiles"][:, 1] = np.arange(B)
        warm["q_tiles"][:, 2] = 1
        for g in range(sizes["n_groups"]):
            warm[f"block_table_{g}"][:] = cache.scratch_page(g)
        self.load(runner, warm)
        runner.model.forward(self.batch, cache)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = runner.model.forward(self.batch, cache)

    def load(self, runner: "StepRunner", arrays) -> None:
        host = runner._stage(self.total)
        for k in self.order:
            a = arrays[k].reshape(-1)
            host[self.offsets[k]:self.offsets[k] + a.size] = a
        self.static.copy_(runner._staging[:self.total], non_blocking=True)
        runner._mark_staged()

    def run(self, runner: "StepRunner", arrays) -> torch.Tensor:
        self.load(runner, arrays)
        self.graph.replay()
        return self.logits


class StepRunner:
    def __init__(self, model: Model, cache: CacheManager, device="cuda:0",
                 decode_graphs: bool = True):
        self.model, self.cache = model, cache
        self.device = torch.device(device)
        self._staging: Optional[torch.Tensor] = None     # pinned host buffer for the tables
        self._staged = None                               # event: last copy out of it is done
        self.steps_run = 0
        # steps made only of single decoded tokens are replayed from captured HIP graphs
        self.decode_graphs = (decode_graphs and self.device.type == "cuda"
                              and getattr(model, "capturable", True))
        self._graphs = {}
        self._graph_seen = {}
        self.graph_replays = 0

    # -- tables to the device ----------------------------------------------------------------
    def _upload(self, arrays) -> dict:
        """All int32 tables in one host-to-device copy; returns views into the device buffer."""
        order = list(arrays)
        offsets, total = {}, 0
        for k in order:
            offsets[k] = total
            total += (arrays[k].size + 3) // 4 * 4        # keep every table 16-byte aligned
        total = max(total, 4)
        host = self._stage(total)
        for k in order:
            a = arrays[k].reshape(-1)
            host[offsets[k]:offsets[k] + a.size] = a
        dev = torch.empty(total, dtype=torch.int32, device=self.device)
        dev.copy_(self._staging[:total], non_blocking=True)
        self._mark_staged()
        return {k: dev[offsets[k]:offsets[k] + arrays[k].size].view(arrays[k].shape)
                for k in order}

    def _stage(self, total: int) -> np.ndarray:
        """The pinned staging buffer as a numpy array of at least ``total`` int32, free to be
        written (the last copy out of it has finished)."""
        if self.device.type != "cuda":
            raise RuntimeError(f"the step function runs on the GPU only, not on {self.device}")
        if self._staging is None or self._staging.numel() < total:
            if self._staged is not None:
                self._staged.synchronize()
            self._staging = torch.empty(max(2 * total, 4096), dtype=torch.int32, pin_memory=True)
            self._staged = None
        if self._staged is not None:
            self._staged.synchronize()
        return self._staging.numpy()

    def _mark_staged(self) -> None:
        self._staged = torch.cuda.Event()
        self._staged.record()

    def make_batch(self, entries: Sequence[StepEntry]) -> RowBatch:
        arrays, sizes = layout_rows(entries, self.cache, self.model.vocab_size)
        dev = self._upload(arrays)
        return RowBatch(
            n_rows=sizes["n_rows"], n_segments=sizes["n_segments"],
            n_logit_rows=sizes["n_logit_rows"], max_position=sizes["max_position"],
            max_segment_rows=sizes["max_segment_rows"],
            tokens=dev["tokens"], row_pos=dev["row_pos"], row_seg=dev["row_seg"],
            seg_start=dev["seg_start"], seg_pos0=dev["seg_pos0"], seg_slot=dev["seg_slot"],
            logit_rows=dev["logit_rows"], q_tiles=dev["q_tiles"],
            block_tables=[dev[f"block_table_{g}"] for g in range(sizes["n_groups"])],
            host=arrays)

    # -- decode steps from captured graphs -----------------------------------------------------
    def _decode_step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Replay the graph for this many single-token segments, capturing it the second time
        its shape is seen.  Returns None when the step should run eagerly.  The logits live in
        the graph's own buffer and are overwritten by its next replay."""
        arrays, sizes = layout_rows(entries, self.cache, self.model.vocab_size)
        ctx_cap = _context_bucket(sizes["max_position"] + 1)
        width = ctx_cap // self.cache.page_size + 1
        for g in range(sizes["n_groups"]):
            bt = arrays[f"block_table_{g}"]
            if bt.shape[1] > width:
                return None
            padded = np.full((bt.shape[0], width), -1, dtype=np.int32)
            padded[:, :bt.shape[1]] = bt
            arrays[f"block_table_{g}"] = padded
        key = (sizes["n_rows"], sizes["n_logit_rows"], ctx_cap)
        graph = self._graphs.get(key)
        if graph is None:
            self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
            if self._graph_seen[key] < 2:
                return None
            if len(self._graphs) >= MAX_DECODE_GRAPHS:
                self._graphs.pop(next(iter(self._graphs)))
            graph = self._graphs[key] = _DecodeGraph(self, arrays, sizes, ctx_cap)
        self.graph_replays += 1
        return graph.run(self, arrays)

    # -- one step ----------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run the entries' tokens as one batch from the cache that earlier steps left and
        return float32 logits [wanted, vocab] on the GPU, in the order of the entries and of
        their ``want``.  If the pages do not suffice, ``OutOfPages`` is raised and neither
        the cache nor any request has changed."""
        entries = list(entries)
        extended: List[StepEntry] = []
        try:
            for e in entries:
                self.cache.extend(e.cache, len(e.tokens))
                extended.append(e)
        except OutOfPages:
            for e in extended:
                self.cache.trim_uncommitted(e.cache)
            raise
        try:
            logits = None
            if self.decode_graphs and all(len(e.tokens) == 1 for e in entries):
                logits = self._decode_step(entries)
            if logits is None:
                batch = self.make_batch(entries)
                logits = self.model.forward(batch, self.cache)
        except Exception:
            for e in entries:
                self.cache.trim_uncommitted(e.cache)
            raise
        for e in entries:
            self.cache.commit(e.cache, len(e.tokens))
        self.steps_run += 1
        return logits
