"""The engine: model, cache, step function, scheduler and sampler behind one object.

kappai's C API is ``engine_init / engine_run / engine_shutdown`` (src/engine.h:12-17) over a
session that prefills in portions and then decodes token by token
(src/context.c:995-1110, 1312-1457), measuring prefill and generation speed with a device
synchronisation before each timestamp (:1507-1512, 1607-1615).  ``Engine`` is the same for
token ids and many requests at once.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..cache.manager import CacheManager
from ..kernels import ops
from ..models import Model, load_model
from ..sampling import RequestSampler, Sampler, SamplingParams
from .batch import StepEntry
from .scheduler import FAILED, RUNNING, Request, Scheduler, SchedulerConfig, TokensUnread
from .step import StepRunner


@dataclass
class EngineConfig:
    """Engine options with kappai's names where it has them (``config``, src/config.h:15-92):
    ``ctx_size`` is -c/--ctx-size (0: from the model)."""
    model: Optional[str] = None          # folder with config.json and model.safetensors
    dtype: str = "bfloat16"
    device: str = "cuda:0"
    ctx_size: int = 0                    # longest sequence; 0: the model's max_position_embeddings
    page_size: int = 16
    num_pages: int = 0                   # 0: from free memory
    memory_fraction: float = 0.8         # share of free GPU memory for pages when num_pages = 0
    max_batch: int = 64                  # requests live at the same time (state slots)
    token_budget: int = 2048
    chunk: int = 2048
    decode_graphs: bool = True           # replay decode steps from captured HIP graphs
    c_forward: bool = True               # steps through the C side (kappai_forward) when the model
                                         # is made of parts it knows
    decode_run: int = 8                  # decode steps queued back to back when nothing but
                                         # decoding is going on (1: every step is waited for)
    pipeline: bool = True                # a step with prompt portions in it is decided and
                                         # queued before the tokens of the step before it have
                                         # been read (they go to their rows on the GPU)
    warm_kernels: bool = True            # run one prompt portion of zeros at start-up, so that
                                         # the first request does not pay for loading the kernels


@dataclass
class Metrics:
    prefill_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_tokens: int = 0
    decode_seconds: float = 0.0
    first_token_ms: float = -1.0
    steps: int = 0

    @property
    def pp(self) -> float:
        return self.prefill_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def tg(self) -> float:
        return self.decode_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0

    def line(self, spec: str = "pp,tg") -> str:
        """kappai's metrics line (src/context.c:1519-1568)."""
        parts = []
        for name in spec.replace(" ", ",").split(","):
            n = name.lower()
            if n == "pp":
                parts.append(f"PP: {self.pp:.2f} t/s")
            elif n == "tg":
                parts.append(f"TG: {self.tg:.2f} t/s")
            elif n == "ttft":
                parts.append(f"TTFT: {self.first_token_ms:.2f} ms" if self.first_token_ms >= 0
                             else "TTFT: --")
        return "[ " + " | ".join(parts) + " ]" if parts else ""


@dataclass
class _TokensOnTheWay:
    """What the sampling kernels of a step (or of a run of decode steps) chose, not read yet: on
    the GPU (for the rows of the step after) and on its way into pinned host memory; ``copied``
    is recorded behind that copy."""
    requests: List[Request]
    place: Dict[int, int]                # id(request) -> its column
    tokens: torch.Tensor                 # int32 [steps * len(requests)] on the GPU, step by step
    host: torch.Tensor                   # pinned, filled when ``copied`` has happened
    copied: "torch.cuda.Event"
    steps: int = 1

    def last(self, request: Request) -> int:
        """Where in ``tokens`` the request's newest token stands."""
        return (self.steps - 1) * len(self.requests) + self.place[id(request)]


@dataclass
class StepOutput:
    request_id: object
    token: Optional[int]
    finished: bool
    finish_reason: Optional[str] = None


class Engine:
    def __init__(self, config: Union[EngineConfig, str, None] = None, model: Optional[Model] = None,
                 **overrides):
        if isinstance(config, str):
            config = EngineConfig(model=config)
        config = config or EngineConfig()
        for k, v in overrides.items():
            if not hasattr(config, k):
                raise TypeError(f"unknown engine option {k!r}")
            setattr(config, k, v)
        self.config = config
        if not torch.cuda.is_available():
            raise RuntimeError("kappai_amd runs on the GPU only and no GPU is visible")
        self.device = torch.device(config.device)
        if model is None:
            if not config.model:
                raise ValueError("an engine needs a model folder (-m/--model)")
            model = load_model(config.model, config.dtype, self.device)
        self.model = model
        mc = model.config
        model_ctx = mc.max_position_embeddings or 0
        self.ctx_size = min(config.ctx_size, model_ctx) if config.ctx_size and model_ctx else (
            config.ctx_size or model_ctx)
        specs = model.cache_specs()
        probe = CacheManager(specs, config.page_size, 1, 1)
        elem = 2 if model.dtype == torch.bfloat16 else 4
        page_bytes = max(probe.bytes_per_token(elem) * config.page_size, 1)
        num_pages = config.num_pages
        if not num_pages:
            free, _ = torch.cuda.mem_get_info(self.device)
            if config.decode_graphs:
                # the captured decode graphs keep logits and workspaces of their own; at most a
                # tenth of the free memory is set aside for them
                free -= min(StepRunner.graph_bytes_bound(mc.vocab_size, config.max_batch),
                            free // 10)
            num_pages = int(free * config.memory_fraction) // page_bytes
            if self.ctx_size:      # no more than every live request at full context
                cap = config.max_batch * ((self.ctx_size + config.page_size - 1) // config.page_size)
                num_pages = min(num_pages, cap)
        if num_pages < 1:
            raise RuntimeError("not enough free GPU memory for a single cache page")
        self.cache = CacheManager(specs, config.page_size, num_pages, config.max_batch)
        self.cache.allocate_storage(model.dtype, self.device)
        self.runner = StepRunner(model, self.cache, self.device,
                                 decode_graphs=config.decode_graphs,
                                 c_forward=config.c_forward)
        eos = mc.eos_token_id
        self.scheduler = Scheduler(
            self.cache,
            SchedulerConfig(config.token_budget, config.chunk, config.max_batch, self.ctx_size),
            eos_token_ids=[] if eos is None else ([eos] if isinstance(eos, int) else eos))
        self.sampler = Sampler()
        self.metrics = Metrics()
        self.requests: Dict[object, Request] = {}
        self._next_id = 0
        self._t_first_add: Optional[float] = None
        self.last_logits: Optional[torch.Tensor] = None
        self.decode_runs = 0              # runs of queued decode steps taken so far
        self.pipelined_steps = 0          # steps queued before their predecessor's tokens were read
        self._on_the_way: List[_TokensOnTheWay] = []
        self._host_ring: List[torch.Tensor] = []
        self._host_at = 0
        if config.warm_kernels:
            self._warm_kernels()

    def _warm_kernels(self) -> None:
        """One prompt portion of the longest size the scheduler will cut, then a single token,
        for a request that is closed again: every kernel a step of that shape needs is loaded and
        has run before the first request arrives (its time to the first token would otherwise
        include that).  Nothing of it is counted in the metrics."""
        pool = min((g.allocator.num_pages for g in self.cache.paged_groups), default=1 << 20)
        n = min(self.config.chunk, self.config.token_budget, pool * self.config.page_size - 1,
                (self.ctx_size or 1 << 30) - 1)
        if n < 1 or self.cache.num_free_slots < 1:
            return
        rc = self.cache.open("warm-up")
        try:
            logits = self.runner.step([StepEntry(rc, [0] * n, [n - 1])])
            warm = RequestSampler(SamplingParams.greedy())
            self.sampler.sample(logits, [warm])
            self.sampler.sample(self.runner.step([StepEntry(rc, [0], [0])]), [warm])
            if self.config.pipeline and n + 3 <= (self.ctx_size or 1 << 30) and \
                    self.cache.can_extend(rc, 2):
                # what a step ahead of its tokens uses beside that: a token placed on the GPU,
                # and the chosen tokens' own way into pinned memory
                chosen = torch.zeros(1, dtype=torch.int32, device=self.device)
                logits = self.runner.step([StepEntry(rc, [0, 0], [1])], placed=(chosen, [(0, 0)]))
                self.sampler.launch(logits, [warm], out=chosen)
                ops.tokens_to_host(chosen, self._pinned(1))
                torch.cuda.synchronize(self.device)
        finally:
            self.cache.close(rc)
        self.runner.steps_run = 0

    # -- requests ----------------------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id=None) -> object:
        params = params or SamplingParams()
        rid = self._next_id if request_id is None else request_id
        if rid in self.requests:
            raise ValueError(f"request id {rid!r} is in use")
        vocab = self.model.vocab_size
        prompt = [int(t) for t in prompt]
        for t in prompt:
            if not 0 <= t < vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        req = Request(rid, prompt, params)
        req.sampler = RequestSampler(params, seed_offset=self._next_id)
        req.sampler.observe(prompt)
        self._next_id += 1
        self.requests[rid] = req
        self.scheduler.add(req)
        if self._t_first_add is None:
            self._t_first_add = time.perf_counter()
        return rid

    def abort(self, request_id) -> bool:
        """Stop a request between two steps: its pages and state slot go back to the pool and
        its output so far stays readable in ``requests[request_id]``.  Returns False when the
        id is unknown or the request had ended already."""
        req = self.requests.get(request_id)
        return req is not None and self.scheduler.abort(req)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished() or bool(self._on_the_way)

    # -- one engine step -----------------------------------------------------------------------
    def _read_tokens(self, records: List[_TokensOnTheWay]) -> List[StepOutput]:
        """Wait for these steps' tokens and hand them to their requests."""
        outputs: List[StepOutput] = []
        for rec in records:
            rec.copied.synchronize()
            width = len(rec.requests)
            tokens = rec.host[:rec.steps * width].tolist()
            if tokens and self.metrics.first_token_ms < 0 and self._t_first_add is not None:
                self.metrics.first_token_ms = (time.perf_counter() - self._t_first_add) * 1e3
            for s in range(rec.steps):
                for req, tok in zip(rec.requests, tokens[s * width:(s + 1) * width]):
                    done = self.scheduler.resolve_token(req, tok)
                    if done is None:
                        continue          # the request had ended before this token
                    req.sampler.observe([tok])
                    outputs.append(StepOutput(req.request_id, tok, done, req.finish_reason))
        return outputs

    def _send_home(self, requests: List[Request], chosen: torch.Tensor, steps: int) -> None:
        """The tokens that kernels already queued will write into ``chosen`` start their way to
        the host, and every request notes how many it has coming."""
        n = chosen.numel()
        host = self._pinned(n)
        ops.tokens_to_host(chosen, host)
        copied = torch.cuda.Event()
        copied.record()
        self._on_the_way.append(_TokensOnTheWay(
            requests, {id(r): i for i, r in enumerate(requests)}, chosen, host, copied, steps))
        for _ in range(steps):
            for r in requests:
                if r.state == RUNNING:    # (it may have reached its count inside the run)
                    self.scheduler.expect_token(r)

    def _read_all(self) -> List[StepOutput]:
        records, self._on_the_way = self._on_the_way, []
        return self._read_tokens(records)

    def _pinned(self, n: int) -> torch.Tensor:
        """The next of a few pinned buffers for token ids on their way to the host."""
        if len(self._host_ring) < 4:
            self._host_ring.append(torch.empty(max(n, self.config.max_batch), dtype=torch.int32,
                                               pin_memory=True))
            return self._host_ring[-1]
        self._host_at = (self._host_at + 1) % len(self._host_ring)
        if self._host_ring[self._host_at].numel() < n:
            self._host_ring[self._host_at] = torch.empty(n, dtype=torch.int32, pin_memory=True)
        return self._host_ring[self._host_at]

    def _can_go_ahead(self, entries, allowed: bool = True) -> bool:
        """Whether this step may be queued before the last step's tokens have been read: every
        token it asks for can be chosen on the GPU, and it holds a prompt portion or is the
        first of a run of decode steps."""
        if not allowed or not self.config.pipeline or not Sampler.runs_on_device(
                [e.request.sampler for e in entries if e.samples], self.model.vocab_size):
            return False
        if any(e.n_tokens > 1 for e in entries):
            return True
        return self._run_length(entries) >= 2

    def _run_length(self, entries) -> int:
        """How many decode steps these entries can take back to back (0: they are not all single
        decoded tokens): nobody may pass its own limits inside the run."""
        n = self.config.decode_run
        if n < 2 or any(e.n_tokens != 1 or not e.samples for e in entries):
            return 0
        for e in entries:
            r = e.request
            if r.params.n_predict >= 0:
                n = min(n, r.params.n_predict - len(r.output))
            n = min(n, self.scheduler.max_context - (len(r.prompt) + len(r.output)))
        return n

    def step(self, go_ahead: bool = True) -> List[StepOutput]:
        """Schedule, run one step of the model, sample, and report every request that got a
        token or ended.  A step that goes ahead of its predecessor's tokens reports those of the
        step before it instead; its own come with the next call.  ``go_ahead=False``: this step
        is waited for."""
        outputs: List[StepOutput] = []
        failed_all: List[Request] = []
        while True:
            try:
                entries, failed = self.scheduler.schedule()
            except TokensUnread:
                if not self._on_the_way:
                    raise
                outputs += self._read_all()
                continue
            failed_all += failed
            ahead = bool(entries) and self._can_go_ahead(entries, go_ahead)
            if ahead or not self._on_the_way:
                break
            outputs += self._read_all()   # the step needs them: read, and decide again
        for req in failed_all:
            outputs.append(StepOutput(req.request_id, None, True, req.finish_reason))
        if not entries:
            return outputs
        if ahead:
            took = self._step_ahead(entries)
            if took is not None:
                return outputs + took
            outputs += self._read_all()   # (no graph for the run yet, or too few pages)
            return outputs + self.step(go_ahead=False)
        run = self._decode_run(entries)
        if run is not None:
            return outputs + run
        t0 = time.perf_counter()          # the last step ended with a synchronisation
        step_entries = []
        for e in entries:
            toks = e.request.tokens_from(e.request.computed, e.n_tokens)
            step_entries.append(StepEntry(e.request.cache, toks,
                                          [e.n_tokens - 1] if e.samples else []))
        logits = self.runner.step(step_entries)
        self.scheduler.advance(entries)
        sampling = [e.request for e in entries if e.samples]
        self.last_logits = logits
        if sampling:                      # reading the tokens back waits for the step
            tokens = self.sampler.sample(logits, [r.sampler for r in sampling],
                                         slots=[r.cache.slot for r in sampling])
        else:
            tokens = []
            torch.cuda.synchronize(self.device)
        self._count(self._tally(entries), time.perf_counter() - t0)
        m = self.metrics
        if tokens and m.first_token_ms < 0 and self._t_first_add is not None:
            m.first_token_ms = (time.perf_counter() - self._t_first_add) * 1e3
        for req, tok in zip(sampling, tokens):
            req.sampler.observe([tok])
            done = self.scheduler.append_token(req, tok)
            outputs.append(StepOutput(req.request_id, tok, done, req.finish_reason))
        return outputs

    @staticmethod
    def _tally(entries):
        """(prompt tokens, decoded tokens) of a step, before its own tokens are recorded."""
        n_prefill = sum(e.n_tokens for e in entries if e.n_tokens > 1 or not e.request.output)
        return n_prefill, sum(e.n_tokens for e in entries) - n_prefill

    def _count(self, tally, dt: float) -> None:
        n_prefill, n_decode = tally
        m = self.metrics
        m.steps += 1
        total = n_prefill + n_decode
        m.prefill_tokens += n_prefill
        m.decode_tokens += n_decode
        m.prefill_seconds += dt * n_prefill / total
        m.decode_seconds += dt * n_decode / total

    def _step_ahead(self, entries) -> List[StepOutput]:
        """Queue the step without having read what the step before it chose: the rows of the
        requests that decode take their tokens from the GPU.  Then wait for the tokens of the
        step before (the GPU is busy with this one meanwhile) and report them."""
        t0 = time.perf_counter()
        newest = self._on_the_way[-1] if self._on_the_way else None
        step_entries, pairs = [], []
        for i, e in enumerate(entries):
            req = e.request
            toks = req.tokens_from(req.computed, e.n_tokens)
            if req.unread:                # the token it goes on from is the newest on the way
                if e.n_tokens != 1 or newest is None or id(req) not in newest.place:
                    raise RuntimeError(f"request {req.request_id!r}: unread tokens out of step")
                toks = [0]
                pairs.append((i, newest.last(req)))
            step_entries.append(StepEntry(req.cache, toks, [e.n_tokens - 1] if e.samples else []))
        run = self._run_length(entries)
        if run >= 2:
            return self._run_ahead(entries, run, newest, pairs, t0)
        logits = self.runner.step(step_entries,
                                  placed=(newest.tokens, pairs) if pairs else None)
        self.scheduler.advance(entries)
        tally = self._tally(entries)
        self.last_logits = logits
        self.pipelined_steps += 1
        older, self._on_the_way = self._on_the_way, []
        sampling = [e.request for e in entries if e.samples]
        if sampling:
            chosen = torch.empty(len(sampling), dtype=torch.int32, device=self.device)
            self.sampler.launch(logits, [r.sampler for r in sampling], out=chosen,
                                slots=[r.cache.slot for r in sampling])
            self._send_home(sampling, chosen, 1)
        outputs = self._read_tokens(older)
        self._count(tally, time.perf_counter() - t0)
        return outputs

    def _run_ahead(self, entries, n: int, newest, pairs, t0) -> Optional[List[StepOutput]]:
        """A run of ``n`` decode steps queued before the tokens on the way have been read: the
        first step takes them on the GPU (``pairs``: (entry, place in ``newest.tokens``)).
        Returns None, with nothing changed, when the run cannot be queued."""
        reqs = [e.request for e in entries]
        samplers = [r.sampler for r in reqs]
        slots = [r.cache.slot for r in reqs]

        def choose(logits, step, out_row, also):
            self.sampler.launch(logits, samplers, out=out_row, also=also, slots=slots)

        first = [0 if r.unread else r.tokens_from(r.computed, 1)[0] for r in reqs]
        tokens = self.runner.decode_run(
            [r.cache for r in reqs], first, n, choose,
            placed=(newest.tokens, pairs) if pairs else None)
        if tokens is None:
            return None
        self.last_logits = None
        self.decode_runs += 1
        self.pipelined_steps += n
        for r in reqs:
            r.computed += n
        older, self._on_the_way = self._on_the_way, []
        self._send_home(reqs, tokens.view(-1), n)
        outputs = self._read_tokens(older)
        m = self.metrics
        m.steps += n
        m.decode_tokens += n * len(reqs)
        m.decode_seconds += time.perf_counter() - t0
        return outputs

    def _decode_run(self, entries) -> Optional[List[StepOutput]]:
        """When every entry is one decoded token, run several steps back to back: each step's
        token goes to the next on the GPU and the host reads them all at the end.  A request
        that meets its end-of-sequence token inside the run has run a few steps too many; they
        are dropped with its cache.  Returns None when the steps have to be taken one by one."""
        n = self._run_length(entries)
        reqs = [e.request for e in entries]
        samplers = [r.sampler for r in reqs]
        if n < 2 or not Sampler.runs_on_device(samplers, self.model.vocab_size):
            return None
        first = [r.tokens_from(r.computed, 1)[0] for r in reqs]
        slots = [r.cache.slot for r in reqs]

        def choose(logits, step, out_row, also):
            self.sampler.launch(logits, samplers, out=out_row, also=also, slots=slots)

        t0 = time.perf_counter()
        tokens = self.runner.decode_run([r.cache for r in reqs], first, n, choose)
        if tokens is None:
            return None
        self.last_logits = None
        self.decode_runs += 1
        rows = tokens.tolist()            # waits for the run
        dt = time.perf_counter() - t0
        m = self.metrics
        m.steps += n
        m.decode_tokens += n * len(reqs)
        m.decode_seconds += dt
        outputs: List[StepOutput] = []
        for row in rows:
            for req, tok in zip(reqs, row):
                if req.state != RUNNING:
                    continue              # ended earlier in the run
                req.computed += 1
                req.sampler.observe([tok])
                done = self.scheduler.append_token(req, tok)
                outputs.append(StepOutput(req.request_id, tok, done, req.finish_reason))
        return outputs

    # -- convenience ---------------------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 on_token=None) -> List[List[int]]:
        """Run the prompts to completion and return the generated token ids of each.  A
        request that fails (it cannot fit the cache) raises."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while self.has_unfinished():
            for out in self.step():
                if on_token is not None and out.token is not None:
                    on_token(out.request_id, out.token)
        result = []
        for rid in ids:
            req = self.requests.pop(rid)
            if req.state == FAILED:
                raise RuntimeError(f"request {rid!r} failed: {req.finish_reason}")
            result.append(list(req.output))
        return result

    def shutdown(self) -> None:
        self._on_the_way.clear()
        for req in list(self.scheduler.running):
            self.scheduler.finish(req, "shutdown")
        self.scheduler.waiting.clear()
        self.requests.clear()
