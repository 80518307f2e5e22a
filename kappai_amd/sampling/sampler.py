"""Choosing the next token of every row of a step's logits.

kappai samples on the host for hybrid models (src/context.c:1318-1319).  Here greedy
choice, the whole-vocabulary temperature draw, the repeat penalty and the draw from
narrowed candidates (top-k, top-p, min-p; kappai's order of operations,
src/sampler.c:218-332) run in HIP kernels on the logits where they lie; the draw's uniform
number comes from the request's own random stream on the host, so that a request's tokens
do not depend on what else is in the batch.  A top-k above 1024 takes a slower kernel that
sorts the whole row in a workspace of its own.

The tokens that the repeat penalty looks at are kept on the GPU as well, a ring per state slot
that the kernels append every chosen token to (``TokenHistory``; kappai's ring on the host:
src/sampler.c:205-216), so that a step with a repeat penalty needs nothing from the host that
the host may not know yet and can be queued ahead like any other.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops, profile
from .params import SamplingParams
from .rng import RandomStream

FILTER_CAP = 1024     # candidates kept when only top-p/min-p narrow (src/sampler.c:7, :225-231)
HISTORY_CAP = 256     # tokens a request's ring on the GPU holds: the longest repeat_last_n that
                      # is served from it (a longer window is applied from the host's list, and
                      # such a step waits for its tokens)


class RequestSampler:
    """Per-request sampling state: options, random stream, and the recent tokens that the
    repeat penalty looks at (prompt included, src/context.c:1513-1514)."""

    def __init__(self, params: SamplingParams, seed_offset: int = 0):
        params.validate()
        self.params = params
        seed = params.seed if params.seed == 0 else params.seed + seed_offset
        self.rng = RandomStream(seed)
        self.recent: List[int] = []

    @property
    def penalised(self) -> bool:
        return self.params.repeat_penalty != 1.0

    @property
    def history_fits(self) -> bool:
        """Whether the window of the repeat penalty fits the ring kept on the GPU."""
        return self.params.repeat_last_n <= HISTORY_CAP

    def observe(self, tokens: Sequence[int]) -> None:
        self.recent.extend(int(t) for t in tokens)
        keep = max(self.params.repeat_last_n, 1)
        if len(self.recent) > 4 * keep:
            del self.recent[:len(self.recent) - keep]

    def penalty_window(self) -> List[int]:
        n = min(self.params.repeat_last_n, len(self.recent))
        return self.recent[len(self.recent) - n:] if n else []


class TokenHistory:
    """The rings of recent tokens on the GPU, one per state slot: ``ring`` [slots, HISTORY_CAP]
    and ``seen`` [slots] (how many tokens went into a ring).  ``owner`` says on the host whose
    history a slot's ring holds: a request that finds another owner there (or none) has its ring
    written anew from the host's list, which is complete whenever that happens (a request gets a
    slot when it is admitted, with every token it has chosen so far read)."""

    def __init__(self, slots: int, device):
        self.ring = torch.zeros((slots, HISTORY_CAP), dtype=torch.int32, device=device)
        self.seen = torch.zeros((slots,), dtype=torch.int32, device=device)
        self.owner = {}


class Sampler:
    """Samples one token for each row of ``logits`` [n, vocab] (float32, on the GPU; changed
    in place where a repeat penalty applies)."""

    RING = 32     # pinned buffers for the per-row numbers of steps that are queued ahead

    def __init__(self):
        self._zeros = {}      # (rows, device) -> zero temperature / uniform tensors (all greedy)
        self._pinned: List[Optional[torch.Tensor]] = [None] * self.RING
        self._pinned_done: List[Optional[torch.cuda.Event]] = [None] * self.RING
        self._ring_at = 0
        self._history: Optional[TokenHistory] = None

    def reserve(self, slots: int, device) -> None:
        """Make the rings for this many state slots now (else they grow when needed)."""
        self._history_for([slots - 1], torch.device(device))

    def _history_for(self, slots: Sequence[int], dev) -> TokenHistory:
        need = max(slots) + 1
        h = self._history
        if h is None or h.ring.shape[0] < need or h.ring.device != dev:
            grown = TokenHistory(max(need, 2 * (h.ring.shape[0] if h is not None else 32)), dev)
            if h is not None and h.ring.device == dev:      # queued work still reads the old one
                grown.ring[:h.ring.shape[0]].copy_(h.ring)
                grown.seen[:h.seen.shape[0]].copy_(h.seen)
                grown.owner = h.owner
            h = self._history = grown
        return h

    def _to_device(self, packed: np.ndarray, dev) -> torch.Tensor:
        """``packed`` (float32) on the GPU through a pinned buffer, without waiting for the GPU."""
        i = self._ring_at
        self._ring_at = (i + 1) % self.RING
        if self._pinned_done[i] is not None:
            self._pinned_done[i].synchronize()
        buf = self._pinned[i]
        if buf is None or buf.numel() < packed.size:
            buf = self._pinned[i] = torch.empty(max(2 * packed.size, 1024), dtype=torch.float32,
                                                pin_memory=True)
        buf.numpy()[:packed.size] = packed
        d = torch.empty(packed.size, dtype=torch.float32, device=dev)
        ops.ints_from_host(buf[:packed.size].view(torch.int32), d.view(torch.int32))
        ev = self._pinned_done[i] = torch.cuda.Event()
        ev.record()
        return d

    @staticmethod
    def runs_on_device(samplers: Sequence[RequestSampler], vocab: int) -> bool:
        """True when every row's token can be chosen without the host seeing the row's earlier
        tokens: no repeat penalty, or one whose window the ring on the GPU holds."""
        return all(not s.penalised or s.history_fits for s in samplers)

    def launch(self, logits: torch.Tensor, samplers: Sequence[RequestSampler],
               out: Optional[torch.Tensor] = None, also: Optional[torch.Tensor] = None,
               slots: Optional[Sequence[int]] = None):
        """Queue the kernels that choose a token for every row; returns the int32 tokens on the
        GPU.  ``also``: a second int32 tensor [rows] that receives them too.  ``slots``: the
        state slot of every row's request, needed when a row has a repeat penalty (its recent
        tokens are kept on the GPU by slot).  Nothing here waits for the GPU."""
        with profile.scope("sample"):
            return self._launch(logits, samplers, out, also, slots)

    def _penalise(self, logits, samplers, slots):
        """Queues the repeat penalty of the rows that have one, from their rings on the GPU, and
        returns what ``_remember`` needs to append the tokens chosen afterwards (or None)."""
        rows = [i for i, s in enumerate(samplers) if s.penalised]
        if not rows:
            return None
        if slots is None or len(slots) != len(samplers):
            raise ValueError("a repeat penalty needs the state slot of every row's request")
        if any(not samplers[i].history_fits for i in rows):
            raise ValueError(f"repeat_last_n above {HISTORY_CAP} is not served from the GPU")
        dev = logits.device
        hist = self._history_for([slots[i] for i in rows], dev)
        fresh = [i for i in rows if hist.owner.get(slots[i]) is not samplers[i]]
        m, f = len(rows), len(fresh)
        windows = [samplers[i].recent[-HISTORY_CAP:] for i in fresh]
        # one copy: [rows | slots | last_n | penalties] of the penalised rows, then, for the
        # rings to write anew, [slots | starts | tokens]
        packed = np.zeros(4 * m + (2 * f + 1 + sum(len(w) for w in windows) if f else 0),
                          dtype=np.float32)
        ints = packed.view(np.int32)
        ints[:m] = rows
        ints[m:2 * m] = [slots[i] for i in rows]
        ints[2 * m:3 * m] = [max(samplers[i].params.repeat_last_n, 0) for i in rows]
        packed[3 * m:4 * m] = [samplers[i].params.repeat_penalty for i in rows]
        if f:
            at = 4 * m
            ints[at:at + f] = [slots[i] for i in fresh]
            starts = np.concatenate([[0], np.cumsum([len(w) for w in windows])])
            ints[at + f:at + 2 * f + 1] = starts
            ints[at + 2 * f + 1:] = [t for w in windows for t in w]
        d = self._to_device(packed, dev)
        di = d.view(torch.int32)
        if f:
            at = 4 * m
            ops.history_set(hist.ring, hist.seen, di[at:at + f], di[at + f:at + 2 * f + 1],
                            di[at + 2 * f + 1:] if di.numel() > at + 2 * f + 1 else di[:0])
            for i in fresh:
                hist.owner[slots[i]] = samplers[i]
        ops.repeat_penalty_history(logits, di[:m], di[m:2 * m], d[3 * m:4 * m], di[2 * m:3 * m],
                                   hist.ring, hist.seen)
        return hist, di[:m], di[m:2 * m]

    @staticmethod
    def _remember(chosen, penalised) -> None:
        if penalised is not None:
            hist, rows, slots = penalised
            ops.history_append(chosen, rows, slots, hist.ring, hist.seen)

    def _launch(self, logits, samplers, out, also=None, slots=None):
        penalised = self._penalise(logits, samplers, slots)
        chosen = self._choose(logits, samplers, out, also)
        self._remember(chosen, penalised)
        return chosen

    def _choose(self, logits, samplers, out, also=None):
        n, vocab = logits.shape
        dev = logits.device
        temps, unis, filt, wide = [], [], [], []
        for i, s in enumerate(samplers):
            p = s.params
            if p.is_greedy():
                temps.append(0.0)
                unis.append(0.0)
            elif p.is_filtered(vocab):
                temps.append(0.0)            # the kernel's choice for this row is replaced
                unis.append(0.0)
                keep = p.top_k if 0 < p.top_k < vocab else min(vocab, FILTER_CAP)
                (filt if keep <= ops.FILTER_MAX_KEEP else wide).append(
                    (i, keep, float(p.temperature), float(p.top_p), float(p.min_p),
                     s.rng.uniform()))
            else:
                temps.append(float(p.temperature))
                unis.append(s.rng.uniform())
        # every per-row number goes to the GPU in ONE copy: [temperature | uniform] for all
        # rows, then [row | keep | temperature | top_p | min_p | uniform] for the narrowed ones
        # (those that keep more than the kernel for narrowed rows holds come last)
        mf = len(filt)
        filt = filt + wide
        m = len(filt)
        if not any(temps) and not m and (n, str(dev)) in self._zeros:
            out_dev = ops.sample_rows(logits, *self._zeros[(n, str(dev))], out=out, also=also)
        else:
            packed = np.zeros(2 * n + 6 * m, dtype=np.float32)
            packed[:n] = temps
            packed[n:2 * n] = unis
            if m:
                cols = list(zip(*filt))
                ints = packed[2 * n:2 * n + 2 * m].view(np.int32)
                ints[:m] = cols[0]
                ints[m:] = cols[1]
                for j in range(4):
                    packed[2 * n + (2 + j) * m:2 * n + (3 + j) * m] = cols[2 + j]
            d = self._to_device(packed, dev)
            if not any(temps) and not m:
                self._zeros[(n, str(dev))] = (d[:n], d[n:2 * n])
            out_dev = ops.sample_rows(logits, d[:n], d[n:2 * n], out=out, also=also)
            if m:
                di = d[2 * n:2 * n + 2 * m].view(torch.int32)
                f = d[2 * n + 2 * m:]
                cols = (di[:m], di[m:], f[:m], f[m:2 * m], f[2 * m:3 * m], f[3 * m:4 * m])
                if mf:
                    ops.sample_filtered(logits, *(c[:mf] for c in cols), out_dev, also=also)
                if m > mf:
                    ops.sample_filtered(logits, *(c[mf:] for c in cols), out_dev, wide=True, also=also)
        return out_dev

    def sample(self, logits: torch.Tensor, samplers: Sequence[RequestSampler],
               slots: Optional[Sequence[int]] = None) -> List[int]:
        """The tokens themselves (waits for the GPU).  With ``slots`` the repeat penalty comes
        from the rings on the GPU as in ``launch``; without them (or with a window longer than a
        ring) from the host's lists, which must then be complete."""
        n, vocab = logits.shape
        if n != len(samplers):
            raise ValueError(f"{n} rows of logits for {len(samplers)} requests")
        if n == 0:
            return []
        dev = logits.device
        if slots is not None and all(s.history_fits for s in samplers if s.penalised):
            return [int(t) for t in self.launch(logits, samplers, slots=slots).tolist()]
        if slots is not None and self._history is not None:
            for slot in slots:        # these tokens do not reach the rings: they are stale now
                self._history.owner.pop(slot, None)
        # repeat penalty from the host's lists: one scatter over all rows that ask for it
        if any(s.params.repeat_penalty != 1.0 and s.recent for s in samplers):
            starts, toks, pens = [0], [], []
            for s in samplers:
                if s.params.repeat_penalty != 1.0:
                    toks.extend(s.penalty_window())
                starts.append(len(toks))
                pens.append(float(s.params.repeat_penalty))
            ops.repeat_penalty(
                logits, torch.tensor(starts, dtype=torch.int32, device=dev),
                torch.tensor(toks or [0], dtype=torch.int32, device=dev),
                torch.tensor(pens, dtype=torch.float32, device=dev))
        return [int(t) for t in self._choose(logits, samplers, None).tolist()]
