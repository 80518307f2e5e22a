"""The scheduler's decisions, without a model: what runs in each step under a token budget,
how prompts are cut, who is admitted, and what happens when pages run out."""
import random

import pytest

from kappai_amd.cache import CacheManager, FixedState, PagedKV
from kappai_amd.engine.scheduler import (FAILED, FINISHED, RUNNING, WAITING, Request, Scheduler,
                                         SchedulerConfig)
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
