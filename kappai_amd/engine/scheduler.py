"""The scheduler: which requests run in the next step, and with how many tokens.

kappai batches requests only in its server: a FIFO queue, a fixed number of live
sessions, prompt portions that run alone and decoded tokens that are coalesced
(src/server/openai.c:1303-1575); its portion sizes come from a heuristic of 32..512 tokens
(src/context.c:937-972).  Here every step has a token budget (2048 by default: a step of
that many rows takes about 6 ms on an MI355X and is the size at which its matrix cores are
used best; 512 rows cost 1.8 times as much per token): each running request that
is decoding gets one token first, then prompts are continued or admitted in arrival
order with portions cut to what is left of the budget.

When pages run out, the request that was admitted last is preempted: everything it holds
is given back and it returns to the front of the queue, to be computed again from its
prompt and the tokens it has generated (state of fixed size cannot be rewound: kappai
poisons an interrupted hybrid session for the same reason, src/context.c:1438-1441).  A
request that cannot fit although it is alone fails with "context exceeds cache".

A step's tokens need not be read back before the next step is decided: ``expect_token`` notes
that a request has a token on the way (its place in ``output`` holds ``UNREAD``), the request
goes on as if that token were no end-of-sequence token, and ``resolve_token`` puts the token
in once it has been read.  What can be known without the token is known at once: a request
that reaches ``n_predict`` or the end of the context with it takes no further step
(``DRAINING``) and ends when the token arrives.  A request whose unread token turns out to be
an end-of-sequence token has run one step too many; that step's token is dropped.  Nothing
that holds unread tokens is preempted or failed: ``schedule`` raises ``TokensUnread`` first,
and the caller reads the tokens and asks again.

The scheduler decides; it runs nothing.  It needs a cache manager's bookkeeping only.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List, Optional, Sequence

from ..cache.manager import CacheManager, RequestCache
from ..sampling.params import SamplingParams

WAITING, RUNNING, FINISHED, FAILED = "waiting", "running", "finished", "failed"
DRAINING = "draining"      # holds its cache, takes no further step, ends when its token is read
UNREAD = -1                # stands in ``Request.output`` for a token that is still on the GPU


class TokensUnread(Exception):
    """A decision needs tokens that have not been read back yet (a request that holds some
    would be preempted or failed).  Nothing has been taken from any request."""


@dataclass
class Request:
    request_id: object
    prompt: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    output: List[int] = field(default_factory=list)
    state: str = WAITING
    finish_reason: Optional[str] = None      # "eos" | "length" | "context" | an error text
    cache: Optional[RequestCache] = None
    computed: int = 0                        # tokens of prompt+output that the cache holds
    admitted_at: int = -1                    # admission counter, for choosing whom to preempt
    preemptions: int = 0
    sampler: object = None                   # per-request sampling state, owned by the engine
    unread: int = 0                          # tokens at the end of ``output`` that are UNREAD
    dropped: int = 0                         # tokens on the way that are to be thrown away
    draining_reason: Optional[str] = None

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    def tokens_from(self, start: int, n: int) -> List[int]:
        """``tokens[start:start + n]`` without putting prompt and output together first."""
        p = len(self.prompt)
        if start >= p:
            return self.output[start - p:start - p + n]
        if start + n <= p:
            return self.prompt[start:start + n]
        return self.prompt[start:] + self.output[:start + n - p]

    @property
    def pending(self) -> int:
        return len(self.prompt) + len(self.output) - self.computed


@dataclass
class Scheduled:
    request: Request
    n_tokens: int
    samples: bool          # the portion ends at the request's last known token: sample after it


@dataclass
class SchedulerConfig:
    token_budget: int = 2048       # tokens a step at most
    chunk: int = 2048              # longest prompt portion
    max_live: int = 64             # requests holding a cache at the same time
    max_context: int = 0           # longest sequence a request may reach (0: pool size)


class Scheduler:
    def __init__(self, cache: CacheManager, config: SchedulerConfig = None,
                 eos_token_ids: Sequence[int] = ()):
        self.cache = cache
        self.config = config or SchedulerConfig()
        if self.config.token_budget < 1 or self.config.chunk < 1:
            raise ValueError("token_budget and chunk must be at least 1")
        self.eos = set(int(t) for t in eos_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self._admissions = 0
        self.preempted_total = 0
        pool_tokens = min((g.allocator.num_pages for g in cache.paged_groups if not g.spec.window),
                          default=10 ** 12) * cache.page_size
        self.max_context = min(self.config.max_context or pool_tokens, pool_tokens)

    # -- queue ---------------------------------------------------------------------------
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise ValueError("a request needs at least one prompt token")
        request.state = WAITING
        self.waiting.append(request)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # -- decisions -----------------------------------------------------------------------
    def _tokens_first(self) -> None:
        """Before room is made at somebody's cost: tokens on the way may end requests and give
        their pages back, and a request that holds some cannot be computed again."""
        for r in self.running:
            if r.unread:
                raise TokensUnread(r.request_id)

    def _preempt(self, victim: Request) -> None:
        self._tokens_first()
        self.cache.close(victim.cache)
        victim.cache = None
        victim.computed = 0
        victim.state = WAITING
        victim.preemptions += 1
        self.preempted_total += 1
        self.running.remove(victim)
        self.waiting.appendleft(victim)

    def _fail(self, request: Request, reason: str, finished: List[Request],
              waiting: bool = False) -> None:
        if not waiting:
            self._tokens_first()
        if request.cache is not None:
            self.cache.close(request.cache)
            request.cache = None
        if request in self.running:
            self.running.remove(request)
        request.state, request.finish_reason = FAILED, reason
        finished.append(request)

    def schedule(self):
        """Returns (entries for the next step, requests that failed while deciding).  If
        requests are live but none of them can go on (their prompts are under way and the
        pool is empty), the one admitted last is preempted, or fails when it is alone, and
        the decision is made again."""
        failed: List[Request] = []
        while True:
            entries = self._schedule_once(failed)
            if entries or not self.running:
                return entries, failed
            self._tokens_first()
            victim = max(self.running, key=lambda r: r.admitted_at)
            if len(self.running) == 1:
                self._fail(victim, "context exceeds cache", failed)
            else:
                self._preempt(victim)

    def _schedule_once(self, failed: List[Request]) -> List[Scheduled]:
        cfg = self.config
        entries: List[Scheduled] = []
        budget = cfg.token_budget
        reserve = [0] * len(self.cache.paged_groups)

        def take(req: Request, n: int) -> bool:
            if not self.cache.can_extend(req.cache, n, reserve):
                return False
            for gi, need in enumerate(self.cache.pages_needed(req.cache, n)):
                reserve[gi] += need
            entries.append(Scheduled(req, n, samples=(n == req.pending)))
            return True

        # 1. one token for every request that is decoding, oldest admission first
        for req in sorted(self.running, key=lambda r: r.admitted_at):
            if req.state != RUNNING or req.pending != 1 or req.computed == 0 or budget < 1:
                continue
            while not take(req, 1):
                self._tokens_first()
                victim = max(self.running, key=lambda r: r.admitted_at)
                if victim is req and len(self.running) == 1:
                    self._fail(req, "context exceeds cache", failed)
                    break
                scheduled = [e for e in entries if e.request is victim]
                if scheduled:       # give its reservation back before it is preempted
                    for e in scheduled:
                        for gi, need in enumerate(self.cache.pages_needed(victim.cache, e.n_tokens)):
                            reserve[gi] -= need
                        entries.remove(e)
                        budget += e.n_tokens
                self._preempt(victim)
                if victim is req:
                    break
            else:
                budget -= 1

        # 2. prompts that are under way, in admission order
        for req in sorted(self.running, key=lambda r: r.admitted_at):
            if budget < 1:
                break
            if any(e.request is req for e in entries) or req.pending < 1 or req.state != RUNNING:
                continue
            n = min(req.pending, cfg.chunk, budget)
            if take(req, n):
                budget -= n

        # 3. admissions in arrival order; the first that does not fit stops them
        while self.waiting and budget >= 1 and len(self.running) < cfg.max_live:
            req = self.waiting[0]
            total = len(req.prompt) + len(req.output)
            if total > self.max_context:
                self.waiting.popleft()
                self._fail(req, "context exceeds cache", failed, waiting=True)
                continue
            if self.cache.num_free_slots < 1:
                break
            n = min(req.pending, cfg.chunk, budget)
            probe = RequestCache(None, -1, len(self.cache.paged_groups))
            if not self.cache.can_extend(probe, n, reserve):
                if not self.running and not entries:
                    self.waiting.popleft()
                    self._fail(req, "context exceeds cache", failed, waiting=True)
                    continue
                break
            self.waiting.popleft()
            req.cache = self.cache.open(req.request_id)
            req.state = RUNNING
            req.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(req)
            take(req, n)
            budget -= n
        return entries

    # -- after the step ------------------------------------------------------------------
    def advance(self, entries: Sequence[Scheduled]) -> None:
        """The step has run: its tokens are in the cache."""
        for e in entries:
            e.request.computed += e.n_tokens

    def _end_by_count(self, request: Request) -> Optional[str]:
        if 0 <= request.params.n_predict <= len(request.output):
            return "length"
        if len(request.prompt) + len(request.output) >= self.max_context:
            return "context"
        return None

    def append_token(self, request: Request, token: int) -> bool:
        """Record a sampled token.  Returns True when the request has finished (its cache is
        given back): end-of-sequence token, ``n_predict`` reached, or the context is full
        (kappai: src/context.c:1332-1334, 1399, 1444-1448)."""
        request.output.append(int(token))
        reason = "eos" if int(token) in self.eos else self._end_by_count(request)
        if reason is None:
            return False
        self.finish(request, reason)
        return True

    def expect_token(self, request: Request) -> None:
        """A token has been chosen for the request on the GPU and not been read yet."""
        request.output.append(UNREAD)
        request.unread += 1
        reason = self._end_by_count(request)
        if reason is not None:
            request.state, request.draining_reason = DRAINING, reason

    def resolve_token(self, request: Request, token: int) -> Optional[bool]:
        """The oldest unread token of the request has arrived.  Returns None when the token is
        one to be thrown away (the request had ended before it), else whether the request has
        finished with it."""
        if request.dropped:
            request.dropped -= 1
            return None
        if request.unread < 1:
            raise ValueError(f"request {request.request_id!r} expects no token")
        at = len(request.output) - request.unread
        request.output[at] = int(token)
        request.unread -= 1
        if int(token) in self.eos:
            request.dropped = request.unread      # steps taken past the end
            del request.output[at + 1:]
            request.unread = 0
            self.finish(request, "eos")
            return True
        if request.state == DRAINING and request.unread == 0:
            self.finish(request, request.draining_reason)
            return True
        return False

    def finish(self, request: Request, reason: str) -> None:
        if request.unread:                        # ended from outside with tokens on the way
            del request.output[len(request.output) - request.unread:]
            request.dropped += request.unread
            request.unread = 0
        if request.cache is not None:
            self.cache.close(request.cache)
            request.cache = None
        if request in self.running:
            self.running.remove(request)
        request.state, request.finish_reason = FINISHED, reason

    def abort(self, request: Request, reason: str = "aborted") -> bool:
        """Take a request out, whether it waits or runs (kappai's interrupt: src/context.c:
        1438-1441; a session with fixed-size state cannot be taken up again afterwards, so
        what it holds is simply given back).  Returns False if it had ended before."""
        if request.state in (FINISHED, FAILED):
            return False
        if request in self.waiting:
            self.waiting.remove(request)
        self.finish(request, reason)
        return True
