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


class StepRunner:
    def __init__(self, model: Model, cache: CacheManager, device="cuda:0"):
        self.model, self.cache = model, cache
        self.device = torch.device(device)
        self._staging: Optional[torch.Tensor] = None     # pinned host buffer for the tables
        self._staged = None                               # event: last copy out of it is done
        self.steps_run = 0

    # -- tables to the device ----------------------------------------------------------------
    def _upload(self, arrays) -> dict:
        """All int32 tables in one host-to-device copy; returns views into the device buffer."""
        order = list(arrays)
        offsets, total = {}, 0
        for k in order:
            offsets[k] = total
            total += (arrays[k].size + 3) // 4 * 4        # keep every table 16-byte aligned
        total = max(total, 4)
        if self.device.type != "cuda":
            raise RuntimeError(f"the step function runs on the GPU only, not on {self.device}")
        if self._staging is None or self._staging.numel() < total:
            self._staging = torch.empty(max(total, 4096), dtype=torch.int32, pin_memory=True)
            self._staged = None
        if self._staged is not None:
            self._staged.synchronize()
        host = self._staging.numpy()
        for k in order:
            a = arrays[k].reshape(-1)
            host[offsets[k]:offsets[k] + a.size] = a
        dev = torch.empty(total, dtype=torch.int32, device=self.device)
        dev.copy_(self._staging[:total], non_blocking=True)
        self._staged = torch.cuda.Event()
        self._staged.record()
        return {k: dev[offsets[k]:offsets[k] + arrays[k].size].view(arrays[k].shape)
                for k in order}

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
