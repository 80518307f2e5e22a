"""The scheduler's decisions, without a model: what runs in each step under a token budget,
how prompts are cut, who is admitted, and what happens when pages run out."""
import random

import pytest

from kappai_amd.cache import CacheManager, FixedState, PagedKV
from kappai_amd.engine.scheduler import (DRAINING, FAILED, FINISHED, RUNNING, UNREAD, WAITING,
                                         Request, Scheduler, SchedulerConfig, TokensUnread)
from kappai_amd.sampling import SamplingParams

SPECS = [FixedState((8, 2)), PagedKV(2, 16), FixedState((8, 2)), PagedKV(2, 16)]


def make(pages=64, slots=8, page_size=4, **cfg):
    cm = CacheManager(SPECS, page_size, pages, slots)
    return cm, Scheduler(cm, SchedulerConfig(**cfg), eos_token_ids=[99])


def req(rid, n_prompt, n_predict=-1):
    return Request(rid, list(range(1, n_prompt + 1)), SamplingParams.greedy(n_predict))


def run_step(cm, sch, next_token=lambda r: 7):
    """Pretend to run a step: take the pages, commit, and give every sampling request a
    token.  Returns (entries, failed, finished)."""
    entries, failed = sch.schedule()
    for e in entries:
        cm.extend(e.request.cache, e.n_tokens)
    for e in entries:
        cm.commit(e.request.cache, e.n_tokens)
    sch.advance(entries)
    finished = [e.request for e in entries if e.samples and sch.append_token(e.request, next_token(e.request))]
    cm.check()
    return entries, failed, finished


def test_prompt_is_cut_under_the_budget():
    cm, sch = make(token_budget=10, chunk=6)
    sch.add(req("a", 20))
    sizes, samples = [], []
    for _ in range(4):
        entries, _, _ = run_step(cm, sch)
        sizes.append([e.n_tokens for e in entries])
        samples.append([e.samples for e in entries])
    assert sizes == [[6], [6], [6], [2]]
    assert samples == [[False], [False], [False], [True]]
    entries, _, _ = run_step(cm, sch)
    assert [(e.n_tokens, e.samples) for e in entries] == [(1, True)]      # now it decodes


def test_decoding_comes_first_then_prompts_in_arrival_order():
    cm, sch = make(token_budget=8, chunk=8)
    sch.add(req("a", 3))
    sch.add(req("b", 9))
    sch.add(req("c", 5))
    e1, _, _ = run_step(cm, sch)
    assert [(e.request.request_id, e.n_tokens) for e in e1] == [("a", 3), ("b", 5)]
    e2, _, _ = run_step(cm, sch)        # a decodes, b goes on, c gets what is left
    assert [(e.request.request_id, e.n_tokens, e.samples) for e in e2] == [
        ("a", 1, True), ("b", 4, True), ("c", 3, False)]
    e3, _, _ = run_step(cm, sch)
    assert [(e.request.request_id, e.n_tokens, e.samples) for e in e3] == [
        ("a", 1, True), ("b", 1, True), ("c", 2, True)]


def test_admission_needs_a_slot_and_keeps_arrival_order():
    cm, sch = make(slots=2, token_budget=64)
    for name in "abc":
        sch.add(req(name, 4, n_predict=2))
    e1, _, _ = run_step(cm, sch)
    assert [e.request.request_id for e in e1] == ["a", "b"]
    assert [r.request_id for r in sch.waiting] == ["c"]
    _, _, fin = run_step(cm, sch)       # a and b reach n_predict = 2 and end
    assert {r.request_id for r in fin} == {"a", "b"} and all(r.finish_reason == "length" for r in fin)
    e3, _, _ = run_step(cm, sch)
    assert [e.request.request_id for e in e3] == ["c"]
    assert cm.num_free_slots == 1


def test_max_live():
    cm, sch = make(token_budget=64, max_live=1)
    sch.add(req("a", 4, n_predict=1))
    sch.add(req("b", 4, n_predict=1))
    e1, _, fin = run_step(cm, sch)
    assert [e.request.request_id for e in e1] == ["a"] and fin[0].request_id == "a"
    e2, _, _ = run_step(cm, sch)
    assert [e.request.request_id for e in e2] == ["b"]


def test_eos_and_context_limit():
    cm, sch = make(token_budget=64, max_context=6)
    sch.add(req("a", 4))
    sch.add(req("b", 4))
    _, _, fin = run_step(cm, sch, next_token=lambda r: 99 if r.request_id == "a" else 5)
    assert [(r.request_id, r.finish_reason) for r in fin] == [("a", "eos")]
    _, _, fin = run_step(cm, sch)       # b: 4 + 2 tokens = the context of 6
    assert [(r.request_id, r.finish_reason) for r in fin] == [("b", "context")]
    assert cm.num_free_pages() == 64
    sch.add(req("long", 7))
    _, failed, _ = run_step(cm, sch)
    assert [(r.request_id, r.state, r.finish_reason) for r in failed] == [
        ("long", FAILED, "context exceeds cache")]


def test_preemption_when_pages_run_out():
    """Three pages of 4 tokens.  a (4 tokens) and b (4 tokens) are admitted; when both need a
    second page, only one is there: b, admitted last, is preempted, gives everything back,
    waits at the front of the queue and is computed again from its prompt and its output."""
    cm, sch = make(pages=3, token_budget=64)
    sch.add(req("a", 4, n_predict=6))
    sch.add(req("b", 4, n_predict=6))
    run_step(cm, sch)
    assert cm.num_free_pages() == 1
    a, b = sch.running
    e2, _, _ = run_step(cm, sch)        # a takes the last page; b cannot and is preempted
    assert [e.request.request_id for e in e2] == ["a"]
    assert b.state == WAITING and b.cache is None and b.computed == 0 and b.preemptions == 1
    assert list(sch.waiting)[0] is b and len(b.output) == 1
    assert cm.num_free_pages() == 1     # b's page came back, a took one
    # b cannot come back while a holds two pages and b needs two (5 tokens): it waits
    for _ in range(4):
        entries, failed, fin = run_step(cm, sch)
        assert not failed
        if fin:
            break
        assert [e.request.request_id for e in entries] == ["a"]
    assert a.state == FINISHED and len(a.output) == 6
    e, _, _ = run_step(cm, sch)         # b is computed again: prompt + its one token, then samples
    assert [(x.request.request_id, x.n_tokens, x.samples) for x in e] == [("b", 5, True)]
    assert len(b.output) == 2
    while sch.has_unfinished():
        run_step(cm, sch)
    assert b.state == FINISHED and len(b.output) == 6
    assert cm.num_free_pages() == 3 and cm.num_free_slots == 8


def test_abort_gives_everything_back_and_lets_the_next_in():
    """A request is taken out while it runs, another while it waits: pages and slot of the
    first go back at once, the one behind them is admitted in the next step, and a second
    abort of the same request changes nothing."""
    cm, sch = make(pages=8, slots=1, page_size=4, token_budget=8, chunk=8)
    a, b, c = req("a", 6), req("b", 5), req("c", 4)
    for r in (a, b, c):
        sch.add(r)
    run_step(cm, sch)
    assert a.state == RUNNING and b.state == WAITING
    free_before = cm.paged_groups[0].allocator.num_free
    assert sch.abort(a) and a.state == FINISHED and a.finish_reason == "aborted"
    assert a.cache is None and cm.num_free_slots == 1
    assert cm.paged_groups[0].allocator.num_free > free_before
    assert sch.abort(b) and b not in sch.waiting
    assert not sch.abort(a) and not sch.abort(b)
    cm.check()
    entries, failed, _ = run_step(cm, sch)
    assert [e.request.request_id for e in entries] == ["c"] and not failed
    assert sch.has_unfinished()


def test_a_request_that_cannot_fit_alone_fails():
    cm, sch = make(pages=2, token_budget=64)
    sch.add(req("big", 9))              # 3 pages needed, the pool has 2: over max_context
    _, failed, _ = run_step(cm, sch)
    assert [r.finish_reason for r in failed] == ["context exceeds cache"]
    sch.add(req("grows", 8))            # fits exactly; the first generated token needs a third page
    _, failed, fin = run_step(cm, sch)
    assert not failed and fin and fin[0].finish_reason == "context"
    assert cm.num_free_pages() == 2


def test_prompts_under_way_cannot_starve_each_other():
    """Two long prompts that together exceed the pool: the one admitted last is preempted so
    that the first can finish; then it runs."""
    cm, sch = make(pages=6, token_budget=8, chunk=8)
    sch.add(req("a", 20, n_predict=1))
    sch.add(req("b", 20, n_predict=1))
    order = []
    for _ in range(40):
        if not sch.has_unfinished():
            break
        entries, failed, fin = run_step(cm, sch)
        assert not failed
        order.extend(r.request_id for r in fin)
    assert order == ["a", "b"]
    assert cm.num_free_pages() == 6


@pytest.mark.parametrize("seed", range(6))
def test_random_load_always_ends(seed):
    rng = random.Random(seed)
    cm, sch = make(pages=rng.randint(6, 30), slots=rng.randint(1, 6), page_size=rng.choice([1, 4, 16]),
                   token_budget=rng.choice([4, 16, 64]), chunk=rng.choice([3, 8, 64]))
    reqs = [req(f"r{i}", rng.randint(1, 30), n_predict=rng.randint(1, 12)) for i in range(25)]
    pending = list(reqs)
    steps = 0
    while pending or sch.has_unfinished():
        if pending and rng.random() < 0.5:
            sch.add(pending.pop(0))
        entries, failed, fin = run_step(cm, sch)
        assert sum(e.n_tokens for e in entries) <= sch.config.token_budget
        assert len({id(e.request) for e in entries}) == len(entries)
        steps += 1
        assert steps < 5000
    for r in reqs:
        assert r.state in (FINISHED, FAILED)
        if r.state == FINISHED:
            assert len(r.output) == r.params.n_predict or r.finish_reason == "context"
        else:
            assert r.finish_reason == "context exceeds cache"
    assert cm.num_free_pages() == cm.paged_groups[0].allocator.num_pages
    assert cm.num_free_slots == cm.num_slots


# ---- tokens that are read a step late ------------------------------------------------------
class Lagged:
    """Drives the scheduler the way an engine does that queues a step before it has read the
    tokens of the step before: ``expect_token`` after each step, ``resolve_token`` a step later
    (or at once, when the scheduler asks for the tokens)."""

    def __init__(self, cm, sch, token_of):
        self.cm, self.sch, self.token_of = cm, sch, token_of
        self.on_the_way = []             # requests whose tokens have not been read, by step
        self.asked = 0                   # times the scheduler wanted the tokens first
        self.dropped = 0

    def read(self, steps):
        finished = []
        for requests in steps:
            for r in requests:
                if r.dropped:
                    done = self.sch.resolve_token(r, 12345)
                    assert done is None
                    self.dropped += 1
                    continue
                at = len(r.output) - r.unread
                if self.sch.resolve_token(r, self.token_of(r, at)):
                    finished.append(r)
        return finished

    def step(self):
        finished = []
        while True:
            try:
                entries, failed = self.sch.schedule()
                break
            except TokensUnread:
                assert self.on_the_way
                self.asked += 1
                steps, self.on_the_way = self.on_the_way, []
                finished += self.read(steps)
        for e in entries:
            self.cm.extend(e.request.cache, e.n_tokens)
        for e in entries:
            self.cm.commit(e.request.cache, e.n_tokens)
        self.sch.advance(entries)
        older, self.on_the_way = self.on_the_way, []
        sampling = [e.request for e in entries if e.samples]
        if sampling:
            self.on_the_way.append(sampling)
            for r in sampling:
                self.sch.expect_token(r)
        finished += self.read(older)
        self.cm.check()
        return entries, failed, finished

    def unfinished(self):
        return self.sch.has_unfinished() or bool(self.on_the_way)


def test_tokens_read_a_step_late():
    """a's third token is the end-of-sequence token.  Read a step late, it is known only after
    a has taken one step more; that step's token is thrown away.  b ends by its count, which is
    known without its token: it takes no step too many."""
    cm, sch = make(token_budget=64)
    lag = Lagged(cm, sch, lambda r, at: 99 if (r.request_id, at) == ("a", 2) else 10 + at)
    a, b = req("a", 4), req("b", 6, n_predict=2)
    sch.add(a)
    sch.add(b)
    e, _, fin = lag.step()               # prompts; nothing read yet
    assert [(x.request.request_id, x.n_tokens) for x in e] == [("a", 4), ("b", 6)] and not fin
    assert a.output == [UNREAD] and a.unread == 1 and a.pending == 1
    e, _, fin = lag.step()               # both decode from tokens they have not seen
    assert [(x.request.request_id, x.n_tokens, x.samples) for x in e] == [
        ("a", 1, True), ("b", 1, True)]
    assert a.output == [10, UNREAD] and b.output == [10, UNREAD]
    assert b.state == DRAINING and not fin       # b's second token is its last, whatever it is
    e, _, fin = lag.step()
    assert [x.request.request_id for x in e] == ["a"]
    assert [(r.request_id, r.finish_reason) for r in fin] == [("b", "length")]
    assert b.output == [10, 11] and b.cache is None
    e, _, fin = lag.step()               # a runs once more while its end token is on the way
    assert [x.request.request_id for x in e] == ["a"]
    assert [(r.request_id, r.finish_reason) for r in fin] == [("a", "eos")]
    assert a.output == [10, 11, 99] and a.dropped == 1 and a.cache is None
    assert lag.unfinished()              # the token of the step too many is still on the way
    e, _, fin = lag.step()
    assert not e and not fin and lag.dropped == 1 and not lag.unfinished()
    assert cm.num_free_pages() == 64 and cm.num_free_slots == 8


def test_nobody_with_unread_tokens_is_preempted():
    """Three pages of 4 tokens; a and b hold one each and both need a second.  With their
    tokens on the way the scheduler asks for the tokens instead of preempting b; once they are
    in, b is preempted with an output that holds no placeholder."""
    cm, sch = make(pages=3, token_budget=64)
    lag = Lagged(cm, sch, lambda r, at: 10 + at)
    a, b = req("a", 4, n_predict=6), req("b", 4, n_predict=6)
    sch.add(a)
    sch.add(b)
    lag.step()
    assert a.unread == 1 and b.unread == 1 and lag.asked == 0
    with pytest.raises(TokensUnread):
        sch.schedule()
    assert a.state == RUNNING and b.state == RUNNING and b.cache is not None   # nothing taken
    e, _, _ = lag.step()
    assert lag.asked == 1 and [x.request.request_id for x in e] == ["a"]
    assert b.state == WAITING and b.output == [10] and b.unread == 0 and b.preemptions == 1
    while lag.unfinished():
        lag.step()
    assert a.output == [10 + i for i in range(6)] and b.output == a.output
    assert cm.num_free_pages() == 3


def test_abort_with_a_token_on_the_way():
    cm, sch = make(token_budget=64)
    lag = Lagged(cm, sch, lambda r, at: 10 + at)
    a = req("a", 4)
    sch.add(a)
    lag.step()
    lag.step()
    assert a.output == [10, UNREAD]
    assert sch.abort(a)
    assert a.output == [10] and a.dropped == 1 and a.unread == 0 and a.cache is None
    _, _, fin = lag.step()
    assert not fin and lag.dropped == 1 and not lag.unfinished()


@pytest.mark.parametrize("seed", range(6))
def test_random_load_read_late_gives_the_same_tokens(seed):
    """The same load with tokens read at once and read a step late: every request ends the same
    way with the same output, whatever was preempted on the way."""
    def token_of(r, at):
        h = hash((r.request_id, at)) % 97
        return 99 if h < 4 else h        # now and then an end-of-sequence token

    def load(lagged):
        rng = random.Random(seed)
        cm, sch = make(pages=rng.randint(6, 30), slots=rng.randint(1, 6),
                       page_size=rng.choice([1, 4, 16]), token_budget=rng.choice([4, 16, 64]),
                       chunk=rng.choice([3, 8, 64]))
        reqs = [req(f"r{i}", rng.randint(1, 30), n_predict=rng.randint(1, 12)) for i in range(25)]
        pending = list(reqs)
        lag = Lagged(cm, sch, token_of)
        steps = 0
        while pending or (lag.unfinished() if lagged else sch.has_unfinished()):
            if pending and rng.random() < 0.5:
                sch.add(pending.pop(0))
            if lagged:
                entries, _, _ = lag.step()
            else:
                entries, _, _ = run_step(cm, sch, next_token=lambda r: token_of(r, len(r.output)))
            assert sum(e.n_tokens for e in entries) <= sch.config.token_budget
            steps += 1
            assert steps < 5000
        assert cm.num_free_pages() == cm.paged_groups[0].allocator.num_pages
        assert cm.num_free_slots == cm.num_slots
        return [(r.state, r.finish_reason, list(r.output)) for r in reqs], lag

    at_once, _ = load(False)
    late, lag = load(True)
    assert late == at_once
    assert all(UNREAD not in out for _, _, out in late)


def test_decode_graphs_are_dropped_in_order_of_last_use():
    """The step function keeps a bounded number of captured decode graphs; the one it drops for a
    new shape is the one used longest ago, and the memory set aside for them is bounded."""
    from kappai_amd.engine.step import MAX_DECODE_GRAPHS, StepRunner

    runner = StepRunner.__new__(StepRunner)
    runner._graphs = {("a",): 1, ("b",): 2, ("c",): 3}
    assert runner._used_graph(("a",)) == 1
    assert list(runner._graphs) == [("b",), ("c",), ("a",)]
    assert runner._used_graph(("nobody",)) is None and len(runner._graphs) == 3
    assert next(iter(runner._graphs)) == ("b",)          # what the next capture would drop
    bound = StepRunner.graph_bytes_bound(65536, 60)      # 60 rows run in the graph of 64
    assert bound == int(MAX_DECODE_GRAPHS * 64 * 65536 * 4 * 1.25)
