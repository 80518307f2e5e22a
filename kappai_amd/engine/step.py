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

from ..cache.manager import CacheManager, OutOfPages, RequestCache
from ..kernels import ops, profile
from ..models.base import Model
from .batch import HostStep, RowBatch, StepEntry, build_step_tables, layout_rows
from .cforward import CForward, NotDescribed, Workspace


CONTEXT_BUCKET_MIN = 1024     # decode graphs are captured for contexts up to a power of two
DECODE_RING = 8            # decode steps whose tables can be queued ahead of the GPU
MAX_DECODE_GRAPHS = 48


# A decode step of B requests that all want logits is replayed from the graph of the next
# batch size in this list, the rows beyond B being dummies on the scratch page and slot: a few
# shapes serve every batch size, and a batch that shrinks as requests end needs no new capture.
DECODE_BATCH_BUCKETS = (1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256)


def _batch_bucket(n_rows: int) -> int:
    for b in DECODE_BATCH_BUCKETS:
        if b >= n_rows:
            return b
    return n_rows


def _context_bucket(n_positions: int) -> int:
    cap = CONTEXT_BUCKET_MIN
    while cap < n_positions:
        cap *= 2
    return cap


class _DecodeGraph:
    """One captured HIP graph of the model's forward pass for B single-token segments whose
    positions lie below ``ctx_cap``: static row tables that every step overwrites, a static
    logits tensor that every replay fills.  The host keeps a mirror of the tables and rewrites
    only what changes from step to step (a block-table row only when its request's pages
    changed)."""

    def __init__(self, runner: "StepRunner", B: int, n_logit: int, ctx_cap: int):
        cache = runner.cache
        n_groups = len(cache.paged_groups)
        self.B, self.n_logit, self.width = B, n_logit, ctx_cap // cache.page_size + 1
        shapes = [("tokens", (B,)), ("row_pos", (B,)), ("row_seg", (B,)), ("seg_start", (B + 1,)),
                  ("seg_pos0", (B,)), ("seg_slot", (B,)), ("logit_rows", (n_logit,))]
        # the parts' own tables, as they come out for B single rows
        self.tables = list(runner.step_tables)
        self.sizes = {"n_rows": B, "n_segments": B, "n_logit_rows": n_logit,
                      "max_position": ctx_cap - 1, "max_segment_rows": 1, "n_groups": n_groups,
                      "logits_of_every_row": n_logit == B}
        z = np.zeros(B, dtype=np.int32)
        extra, numbers = build_step_tables(self.tables, HostStep(
            {"tokens": z, "row_pos": z, "row_seg": np.arange(B, dtype=np.int32),
             "seg_start": np.arange(B + 1, dtype=np.int32), "seg_pos0": z, "seg_slot": z,
             "logit_rows": (np.arange(n_logit) % B).astype(np.int32)}, self.sizes,
            cache.page_size))
        self.numbers = numbers
        shapes += [(name, a.shape) for name, a in extra.items()]
        shapes += [("place_dst", (B,)), ("place_src", (B,))]
        shapes += [(f"block_table_{g}", (B, self.width)) for g in range(n_groups)]
        self.offsets, total = {}, 0
        for k, shp in shapes:
            self.offsets[k] = total
            total += (int(np.prod(shp)) + 3) // 4 * 4
        self.total = max(total, 4)
        self.mirror = np.zeros(self.total, dtype=np.int32)
        self.h = {k: self.mirror[self.offsets[k]:self.offsets[k] + int(np.prod(shp))].reshape(shp)
                  for k, shp in shapes}
        dev = runner.device
        self.static = torch.zeros(self.total, dtype=torch.int32, device=dev)
        views = {k: self.static[self.offsets[k]:self.offsets[k] + int(np.prod(shp))].view(shp)
                 for k, shp in shapes}
        self.views = views
        self.batch = RowBatch(
            n_rows=B, n_segments=B, n_logit_rows=n_logit, max_position=ctx_cap - 1,
            max_segment_rows=1, tokens=views["tokens"], row_pos=views["row_pos"],
            row_seg=views["row_seg"], seg_start=views["seg_start"], seg_pos0=views["seg_pos0"],
            seg_slot=views["seg_slot"], logit_rows=views["logit_rows"],
            extra={name: views[name] for name in extra}, numbers=dict(numbers),
            block_tables=[views[f"block_table_{g}"] for g in range(n_groups)], host={},
            logits_of_every_row=n_logit == B)
        # what never changes
        self.h["row_seg"][:] = np.arange(B)
        self.h["seg_start"][:] = np.arange(B + 1)
        for name, a in extra.items():
            self.h[name][...] = a
        # tables that depend on more than the number of rows are built again for every replay
        self.rebuilt = [t for t in self.tables if not t.decode_constant]
        # a warm-up run on the scratch page and the scratch slot: every kernel of this shape is
        # loaded and has run once before the capture, and no request's cache is touched
        self.h["seg_slot"][:] = cache.scratch_slot
        self.h["logit_rows"][:] = np.arange(n_logit) % B
        for g in range(n_groups):
            self.h[f"block_table_{g}"][:] = cache.scratch_page(g)
        self.rows_of = [None] * B        # (request cache, version) whose pages row si mirrors
        self.scratch = (cache.scratch_slot, [cache.scratch_page(g) for g in range(n_groups)])
        self._ring: List[Optional[torch.Tensor]] = [None] * DECODE_RING
        self._ring_done: List[Optional[torch.cuda.Event]] = [None] * DECODE_RING
        self._ring_at = 0
        self._upload(runner)
        # (a workspace of the graph's own: its kernels keep addresses inside it)
        self.workspace = Workspace()
        runner.forward(self.batch, self.workspace)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = runner.forward(self.batch, self.workspace)

    def _upload(self, runner: "StepRunner", keep_tokens: bool = False) -> None:
        """The mirror to the device through the next pinned buffer of the graph's ring, so that
        several steps can be queued before the first of them has run.  ``keep_tokens``: all of it
        but the token table, which kernels queued before have filled on the GPU."""
        i = self._ring_at
        self._ring_at = (i + 1) % len(self._ring)
        if self._ring_done[i] is not None:
            self._ring_done[i].synchronize()
        if self._ring[i] is None:
            self._ring[i] = torch.empty(self.total, dtype=torch.int32, pin_memory=True)
        self._ring[i].numpy()[:] = self.mirror
        first = self.offsets["row_pos"] if keep_tokens else 0      # (the token table comes first)
        ops.ints_from_host(self._ring[i][first:], self.static[first:])
        ev = self._ring_done[i] = torch.cuda.Event()
        ev.record()

    def token_table(self, n: int) -> torch.Tensor:
        """Where the next replay reads the tokens of its first ``n`` rows."""
        return self.views["tokens"][:n]

    def run(self, runner: "StepRunner", caches, tokens, pos, slots, logit_rows,
            device_tokens: Optional[torch.Tensor] = None, placed=None,
            tokens_in_place: bool = False) -> torch.Tensor:
        """``tokens`` from the host, or ``device_tokens`` (int32 [B] on the GPU, e.g. what the last
        step's sampling kernel wrote) copied into place on the GPU, or the host's with some of
        them replaced on the GPU (``placed``, as in ``StepRunner.step``), or none of these:
        ``tokens_in_place`` says that kernels queued before this call write the tokens into
        ``token_table`` themselves."""
        h = self.h
        if placed is not None:
            for k, (row, at) in enumerate(placed[1]):
                h["place_dst"][k] = row
                h["place_src"][k] = at
        n = len(caches)                  # rows n .. B-1 are dummies: token 0 at position 0 of
        if device_tokens is None and not tokens_in_place:     # the scratch slot and page, logits
            h["tokens"][:n] = tokens                           # nobody reads
        h["tokens"][n:] = 0
        h["row_pos"][:n] = pos
        h["row_pos"][n:] = 0
        h["seg_pos0"][:n] = pos
        h["seg_pos0"][n:] = 0
        h["seg_slot"][:n] = slots
        h["seg_slot"][n:] = self.scratch[0]
        if n < self.B:
            h["logit_rows"][:] = np.arange(self.n_logit) % self.B
        else:
            h["logit_rows"][:] = logit_rows
        for si, rc in enumerate(caches):
            seen = self.rows_of[si]
            if seen is None or seen[0] is not rc or seen[1] != rc.version:
                for g in range(len(rc.blocks)):
                    row = h[f"block_table_{g}"][si]
                    b = rc.block_array(g)
                    row[:b.size] = b
                    row[b.size:] = -1
                self.rows_of[si] = (rc, rc.version)
        for si in range(n, self.B):
            if self.rows_of[si] is not None:
                for g, page in enumerate(self.scratch[1]):
                    h[f"block_table_{g}"][si] = page
                self.rows_of[si] = None
        if self.rebuilt:
            made, nums = build_step_tables(self.rebuilt, HostStep(
                {k: h[k] for k in ("tokens", "row_pos", "row_seg", "seg_start", "seg_pos0",
                                   "seg_slot", "logit_rows")}, self.sizes,
                runner.cache.page_size))
            for name, a in made.items():
                if name not in h or a.shape != h[name].shape:
                    raise RuntimeError(f"the table {name!r} changed its shape between the steps of "
                                       f"a captured graph; its part must not be capturable")
                h[name][...] = a
            if any(self.numbers.get(k) != v for k, v in nums.items()):
                raise RuntimeError("a number that a launch is sized by changed between the steps "
                                   "of a captured graph; its part must not be capturable")
        self._upload(runner, keep_tokens=tokens_in_place)
        if tokens_in_place:
            pass
        elif device_tokens is not None:
            self.batch.tokens[:n].copy_(device_tokens)
        elif placed is not None and placed[1]:
            m = len(placed[1])
            ops.place_tokens(self.batch.tokens, self.views["place_dst"][:m], placed[0],
                             self.views["place_src"][:m])
        self.graph.replay()
        return self.logits if n == self.B else self.logits[:n]


class StepRunner:
    def __init__(self, model: Model, cache: CacheManager, device="cuda:0",
                 decode_graphs: bool = True, c_forward: bool = True):
        """``c_forward``: run steps through the C side (``kappai_forward``) when every part of the
        model describes itself for it; False runs every step from the parts' own ``forward``
        methods."""
        self.model, self.cache = model, cache
        self.device = torch.device(device)
        self.c_forward = c_forward and self.device.type == "cuda"
        self._cplan: Optional[CForward] = None
        self._cplan_tried = False
        self._staging: Optional[torch.Tensor] = None     # pinned host buffer for the tables
        self._staged = None                               # event: last copy out of it is done
        self.steps_run = 0
        # steps made only of single decoded tokens are replayed from captured HIP graphs
        self.decode_graphs = (decode_graphs and self.device.type == "cuda"
                              and getattr(model, "capturable", True))
        self._graphs = {}
        self._graph_seen = {}
        self.graph_replays = 0
        # what the model's parts want laid out beside the step's own tables
        tables = getattr(model, "step_tables", None)
        self.step_tables = list(tables()) if callable(tables) else []

    # -- the forward pass of a step ----------------------------------------------------------
    def forward(self, batch: RowBatch, workspace: Optional[Workspace] = None) -> torch.Tensor:
        """The model over the rows of ``batch``: one call into C when there is a plan for the
        model (made at the first step, when the cache's storage exists) and nobody is timing the
        stages, else part by part from the host."""
        if self.c_forward and not self._cplan_tried:
            self._cplan_tried = True
            if CForward.plannable(self.model):
                try:
                    self._cplan = CForward(self.model, self.cache, self.device)
                except NotDescribed:       # a part without a description for the C side
                    self._cplan = None
        if self._cplan is not None and not profile.STAGE_TIMES.enabled:
            return self._cplan.forward(batch, workspace)
        return self.model.forward(batch, self.cache)

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
        ops.ints_from_host(self._staging[:total], dev)
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

    def make_batch(self, entries: Sequence[StepEntry], placed=None) -> RowBatch:
        """``placed``: see ``step``."""
        arrays, sizes = layout_rows(entries, self.cache, self.model.vocab_size, self.step_tables)
        if placed is not None and placed[1]:
            chosen, pairs = placed
            for ei, at in pairs:
                if not (0 <= ei < len(entries) and 0 <= at < chosen.numel()):
                    raise ValueError(f"placed token: entry {ei} or place {at} does not exist")
            arrays["place_dst"] = arrays["seg_start"][[ei for ei, _ in pairs]]
            arrays["place_src"] = np.asarray([at for _, at in pairs], dtype=np.int32)
        dev = self._upload(arrays)
        if "place_dst" in arrays:
            ops.place_tokens(dev["tokens"], dev["place_dst"], placed[0], dev["place_src"])
        return RowBatch(
            n_rows=sizes["n_rows"], n_segments=sizes["n_segments"],
            n_logit_rows=sizes["n_logit_rows"], max_position=sizes["max_position"],
            max_segment_rows=sizes["max_segment_rows"],
            tokens=dev["tokens"], row_pos=dev["row_pos"], row_seg=dev["row_seg"],
            seg_start=dev["seg_start"], seg_pos0=dev["seg_pos0"], seg_slot=dev["seg_slot"],
            logit_rows=dev["logit_rows"], extra={name: dev[name] for name in sizes["extra"]},
            numbers=sizes["numbers"], logits_of_every_row=sizes["logits_of_every_row"],
            block_tables=[dev[f"block_table_{g}"] for g in range(sizes["n_groups"])],
            host=arrays)

    # -- decode steps from captured graphs -----------------------------------------------------
    def _decode_step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Replay the graph for this many single-token segments, capturing it the second time
        its shape is seen.  Returns None when the step should run eagerly.  The logits live in
        the graph's own buffer and are overwritten by its next replay."""
        B = len(entries)
        caches = [e.cache for e in entries]
        if len({id(c) for c in caches}) != B:
            return None                     # the eager path reports the duplicate
        tokens = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=B)
        if tokens.min() < 0 or tokens.max() >= self.model.vocab_size:
            return None                     # the eager path reports the bad id
        logit_rows = []
        for si, e in enumerate(entries):
            if len(e.want) == 1 and int(e.want[0]) == 0:
                logit_rows.append(si)
            elif len(e.want) != 0:
                return None
        # positions before this step's tokens were made room for: length is not yet committed
        pos = np.fromiter((c.length for c in caches), dtype=np.int32, count=B)
        ctx_cap = _context_bucket(int(pos.max()) + 1)
        width = ctx_cap // self.cache.page_size + 1
        if any(len(b) > width for c in caches for b in c.blocks):
            return None
        # every row wants its logits (the usual decode step): the graph of the next batch size
        rows_b = _batch_bucket(B) if len(logit_rows) == B else B
        n_logit = rows_b if len(logit_rows) == B else len(logit_rows)
        key = (rows_b, n_logit, ctx_cap)
        graph = self._used_graph(key)
        if graph is None:
            self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
            if self._graph_seen[key] < 2:
                return None
            if len(self._graphs) >= MAX_DECODE_GRAPHS:
                self._graphs.pop(next(iter(self._graphs)))     # the one used longest ago
            graph = self._graphs[key] = _DecodeGraph(self, rows_b, n_logit, ctx_cap)
        slots = np.fromiter((c.slot for c in caches), dtype=np.int32, count=B)
        self.graph_replays += 1
        return graph.run(self, caches, tokens, pos, slots, logit_rows)

    def _used_graph(self, key) -> Optional[_DecodeGraph]:
        """The captured graph of this shape, moved to the end of the dictionary: its order is
        the order of last use, so the graph that is dropped when a new shape arrives is the one
        used longest ago, not a hot one."""
        graph = self._graphs.pop(key, None)
        if graph is not None:
            self._graphs[key] = graph
        return graph

    @staticmethod
    def graph_bytes_bound(vocab_size: int, max_batch: int) -> int:
        """An upper bound on the device memory that captured decode graphs hold beside the cache:
        each keeps its own logits [rows, vocab] in float32 and a workspace for its activations
        (taken as a quarter of that again); the rows are the batch bucket of ``max_batch`` at
        most, and ``MAX_DECODE_GRAPHS`` are kept."""
        rows = _batch_bucket(max(1, max_batch))
        return int(MAX_DECODE_GRAPHS * rows * vocab_size * 4 * 1.25)

    def decode_run(self, caches: Sequence[RequestCache], first_tokens: Sequence[int], n_steps: int,
                   choose, out: Optional[torch.Tensor] = None,
                   placed=None) -> Optional[torch.Tensor]:
        """``n_steps`` decode steps of the same requests, queued back to back: the token a step
        chooses goes to the next step on the GPU, and the host does not wait in between.
        ``choose(logits, step, out_row, also)`` queues the kernels that write one token per request
        (int32) into ``out_row`` and, when ``also`` is a tensor, into it as well (the token table
        of the next step: no copy runs between two steps).  Returns the tokens [n_steps, B] on the GPU (not yet waited
        for), or None when the run cannot be made this way (no captured graph for the shape
        yet, not enough pages for all the steps): then nothing has changed.  After the run
        every cache holds ``n_steps`` more tokens.  ``placed`` = (int32 tensor on the GPU, [(request,
        place), ...]): the first token of these requests is the one at that place of the tensor
        (chosen by kernels that are queued already), not the one in ``first_tokens``."""
        B = len(caches)
        if placed is not None:
            for row, at in placed[1]:
                if not (0 <= row < B and 0 <= at < placed[0].numel()):
                    raise ValueError(f"placed token: request {row} or place {at} does not exist")
        if not self.decode_graphs or B == 0 or n_steps < 1 or n_steps > DECODE_RING:
            return None
        if len({id(c) for c in caches}) != B:
            return None
        ctx_cap = _context_bucket(max(c.length for c in caches) + n_steps)
        rows_b = _batch_bucket(B)
        graph = self._used_graph((rows_b, rows_b, ctx_cap))
        if graph is None or not self.cache.can_extend_all(caches, n_steps):
            return None
        tokens = np.asarray(first_tokens, dtype=np.int64)
        if tokens.shape != (B,) or tokens.min() < 0 or tokens.max() >= self.model.vocab_size:
            return None
        if out is None:
            out = torch.empty((n_steps, B), dtype=torch.int32, device=self.device)
        slots = np.fromiter((c.slot for c in caches), dtype=np.int32, count=B)
        rows = list(range(B))
        for s in range(n_steps):
            for c in caches:
                self.cache.extend_one(c)
            pos = np.fromiter((c.length for c in caches), dtype=np.int32, count=B)
            logits = graph.run(self, caches, tokens, pos, slots, rows,
                               placed=placed if s == 0 else None, tokens_in_place=s > 0)
            for c in caches:
                self.cache.commit_one(c)
            choose(logits, s, out[s], graph.token_table(B) if s + 1 < n_steps else None)
            self.graph_replays += 1
            self.steps_run += 1
        return out

    # -- one step ----------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], placed=None) -> torch.Tensor:
        """Run the entries' tokens as one batch from the cache that earlier steps left and
        return float32 logits [wanted, vocab] on the GPU, in the order of the entries and of
        their ``want``.  If the pages do not suffice, ``OutOfPages`` is raised and neither
        the cache nor any request has changed.

        ``placed`` = (int32 tensor on the GPU, [(entry, place), ...]): the first token of each
        of these entries is not the one in its ``tokens`` but the one at that place of the
        tensor, which the GPU has or will have when the step runs (what sampling kernels wrote
        for the step before, not read back yet)."""
        entries = list(entries)
        if not entries:
            raise ValueError("a step needs at least one entry")
        single = all(len(e.tokens) == 1 for e in entries) and placed is None
        extended: List[StepEntry] = []
        try:
            for e in entries:
                if single:
                    self.cache.extend_one(e.cache)
                else:
                    self.cache.extend(e.cache, len(e.tokens))
                extended.append(e)
        except OutOfPages:
            for e in extended:
                self.cache.trim_uncommitted(e.cache)
            raise
        try:
            logits = None
            if self.decode_graphs and single:
                logits = self._decode_step(entries)
            if logits is None:
                batch = self.make_batch(entries, placed)
                logits = self.forward(batch)
        except Exception:
            for e in entries:
                self.cache.trim_uncommitted(e.cache)
            raise
        for e in entries:
            if single:
                self.cache.commit_one(e.cache)
            else:
                self.cache.commit(e.cache, len(e.tokens))
        self.steps_run += 1
        return logits
