"""The host side of the C API (``csrc/engine_api.h``).

kappai's entry points are C: ``engine_init_config / engine_run / engine_shutdown``
(src/engine.h:12-17) over a session (src/context.h:100-137).  Here the engine is Python, and the C
library ``engine_api`` is a shell over it: it holds an interpreter (its own, or the one of the
process that loaded it), creates a ``Session`` through this module and calls its methods with
plain numbers: sizes, request ids and the addresses of the caller's buffers, which are read and
written in place.  Nothing of the engine's logic lives in C or here; a session is an ``Engine``
and, for the raw step function, the engine's own ``StepRunner`` and cache.
"""
from __future__ import annotations

import ctypes
from typing import Dict

import numpy as np

from ..sampling import SamplingParams
from .batch import StepEntry
from .engine import Engine, EngineConfig

# codes of kappai_step_output.reason (csrc/engine_api.h)
FINISH_REASONS = ["", "eos", "length", "context", "failed", "aborted", "shutdown"]


def _ints(address: int, n: int) -> np.ndarray:
    """The caller's ``int[n]`` at ``address`` as an array (no copy)."""
    if n <= 0:
        return np.zeros(0, dtype=np.int32)
    return np.ctypeslib.as_array((ctypes.c_int * n).from_address(address))


class Session:
    def __init__(self, options: dict):
        device = f"cuda:{int(options.pop('device', 0))}"
        config = EngineConfig(device=device)
        for key, value in options.items():
            if not hasattr(config, key):
                raise TypeError(f"unknown engine option {key!r}")
            if isinstance(value, bool) or value not in (None, 0, ""):
                setattr(config, key, value)           # (0 and "" leave the engine's default)
        self.engine = Engine(config)
        self.pending: list = []                      # outputs not handed to the caller yet
        self.raw: Dict[int, object] = {}             # request caches of the raw step function

    # -- requests --------------------------------------------------------------------------------
    def add_request(self, ids_address: int, n: int, temperature: float, top_k: int, top_p: float,
                    min_p: float, repeat_penalty: float, repeat_last_n: int, seed: int,
                    n_predict: int) -> int:
        params = SamplingParams(temperature, top_k, top_p, min_p, repeat_penalty, repeat_last_n,
                                seed, n_predict)
        params.validate()
        return int(self.engine.add_request(_ints(ids_address, n).tolist(), params))

    def abort(self, request_id: int) -> int:
        return 1 if self.engine.abort(request_id) else 0

    def has_work(self) -> int:
        return 1 if (self.pending or self.engine.has_unfinished()) else 0

    def step(self, out_address: int, capacity: int) -> int:
        """One engine step; up to ``capacity`` outputs (request id, token or -1, finished, reason)
        go to the caller's ``int[capacity][4]``; what does not fit waits for the next call."""
        if not self.pending and self.engine.has_unfinished():
            self.pending = list(self.engine.step())
        out = _ints(out_address, 4 * capacity).reshape(capacity, 4) if capacity > 0 else None
        n = min(len(self.pending), max(capacity, 0))
        for i, o in enumerate(self.pending[:n]):
            reason = o.finish_reason or ""
            code = FINISH_REASONS.index(reason) if reason in FINISH_REASONS else (
                4 if o.finished else 0)       # any other text says why the request failed
            out[i] = (int(o.request_id), -1 if o.token is None else int(o.token),
                      1 if o.finished else 0, code)
        self.pending = self.pending[n:]
        return n

    def output(self, request_id: int, out_address: int, capacity: int) -> int:
        """The tokens a request has generated so far; returns their number (which may exceed
        ``capacity``: then only the first ``capacity`` were written)."""
        req = self.engine.requests.get(request_id)
        if req is None:
            raise KeyError(f"no request {request_id}")
        tokens = [t for t in req.output if t >= 0]
        n = min(len(tokens), max(capacity, 0))
        if n:
            _ints(out_address, n)[:] = tokens[:n]
        return len(tokens)

    def release(self, request_id: int) -> int:
        """Forget a request that has ended (its output is no longer kept)."""
        return 1 if self.engine.requests.pop(request_id, None) is not None else 0

    def generate(self, ids_address: int, n: int, temperature: float, top_k: int, top_p: float,
                 min_p: float, repeat_penalty: float, repeat_last_n: int, seed: int,
                 n_predict: int, out_address: int, capacity: int) -> int:
        """Blocking: one prompt to its end; the generated tokens go to ``int[capacity]``."""
        params = SamplingParams(temperature, top_k, top_p, min_p, repeat_penalty, repeat_last_n,
                                seed, n_predict)
        params.validate()
        (tokens,) = self.engine.generate([_ints(ids_address, n).tolist()], params)
        m = min(len(tokens), max(capacity, 0))
        if m:
            _ints(out_address, m)[:] = tokens[:m]
        return len(tokens)

    # -- the raw step function -----------------------------------------------------------------
    def forward(self, n_entries: int, ids_address: int, counts_address: int,
                tokens_address: int, want_counts_address: int, want_address: int,
                logits_address: int, capacity_floats: int) -> int:
        """One step of the engine's own step function over ``n_entries`` (request id, its next
        tokens, the places among them whose logits are wanted), as trace replay drives it: a
        request id not seen before opens a request.  float32 logits [wanted, vocab] go to the
        caller's buffer; returns the number of wanted rows."""
        ids = _ints(ids_address, n_entries)
        counts = _ints(counts_address, n_entries)
        want_counts = _ints(want_counts_address, n_entries)
        tokens = _ints(tokens_address, int(counts.sum()))
        want = _ints(want_address, int(want_counts.sum()))
        cache = self.engine.cache
        entries, at, wat, opened = [], 0, 0, []
        try:
            for rid, n, nw in zip(ids.tolist(), counts.tolist(), want_counts.tolist()):
                if rid not in self.raw:
                    self.raw[rid] = cache.open(("raw", rid))
                    opened.append(rid)
                entries.append(StepEntry(self.raw[rid], tokens[at:at + n].tolist(),
                                         want[wat:wat + nw].tolist()))
                at += n
                wat += nw
            vocab = self.engine.model.vocab_size
            if wat * vocab > capacity_floats:
                raise ValueError(f"{wat} rows of {vocab} logits do not fit {capacity_floats} floats")
            logits = self.engine.runner.step(entries)
        except Exception:
            for rid in opened:
                cache.close(self.raw.pop(rid))
            raise
        if wat:
            dst = np.ctypeslib.as_array(
                (ctypes.c_float * (wat * vocab)).from_address(logits_address)).reshape(wat, vocab)
            dst[:] = logits.detach().to("cpu").numpy()
        return wat

    def end(self, request_id: int) -> int:
        """A request of the raw step function is finished: what it holds is given back."""
        rc = self.raw.pop(request_id, None)
        if rc is None:
            return 0
        self.engine.cache.close(rc)
        return 1

    # -- numbers ---------------------------------------------------------------------------------
    def stats(self, out_address: int, n: int) -> int:
        """double[n]: steps, prompt tokens, prompt seconds, decoded tokens, decode seconds, first
        token ms, graph replays, preemptions, free pages, vocabulary, longest sequence."""
        e, m = self.engine, self.engine.metrics
        free = min((g.allocator.num_free for g in e.cache.paged_groups), default=0)
        values = [m.steps, m.prefill_tokens, m.prefill_seconds, m.decode_tokens, m.decode_seconds,
                  m.first_token_ms, e.runner.graph_replays, e.scheduler.preempted_total, free,
                  e.model.vocab_size, e.ctx_size]
        k = min(n, len(values))
        if k > 0:
            np.ctypeslib.as_array((ctypes.c_double * k).from_address(out_address))[:] = values[:k]
        return len(values)

    def close(self) -> None:
        for rid in list(self.raw):
            self.end(rid)
        self.engine.shutdown()


def create(options: dict) -> Session:
    return Session(dict(options))
