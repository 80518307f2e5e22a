"""The cache manager's bookkeeping: no page lost, held twice or freed twice, under random
orders of requests; groups with their own pools; windows giving pages back."""
import random

import pytest

from kappai_amd.cache import (CacheError, CacheManager, FixedState, OutOfPages, OutOfSlots,
                              PageAllocator, PagedKV)


def specs_lfm2_like():
    full = PagedKV(2, 16)
    conv = FixedState((64, 2))
    return [conv, full, conv, full]


def test_grouping():
    cm = CacheManager(specs_lfm2_like() + [PagedKV(2, 16, window=8), None], 4, 10, 3)
    assert len(cm.paged_groups) == 2 and len(cm.state_groups) == 1
    assert cm.paged_groups[0].cache_ids == [1, 3] and cm.paged_groups[1].cache_ids == [4]
    assert cm.state_groups[0].cache_ids == [0, 2]
    assert cm.view(1).group == 0 and cm.view(4).group == 1 and cm.view(0).group == 0
    with pytest.raises(CacheError):
        cm.view(5)
    assert cm.bytes_per_token(2) == 2 * 2 * 16 * 2 * 3


def test_allocator_refuses_misuse():
    a = PageAllocator(3)
    p = a.take("x")
    with pytest.raises(CacheError, match="belongs"):
        a.give_back(p, "y")
    a.give_back(p, "x")
    with pytest.raises(CacheError, match="freed twice"):
        a.give_back(p, "x")
    with pytest.raises(CacheError, match="does not exist"):
        a.give_back(7, "x")
    got = [a.take("z") for _ in range(3)]
    assert sorted(got) == [0, 1, 2]
    with pytest.raises(OutOfPages):
        a.take("z")
    a.check()


def test_pages_follow_tokens_and_return():
    cm = CacheManager(specs_lfm2_like(), 4, 6, 2)
    a = cm.open("a")
    cm.extend(a, 5)
    assert len(a.blocks[0]) == 2 and cm.num_free_pages() == 4
    cm.commit(a, 5)
    cm.extend(a, 3)                      # 8 tokens: still two pages
    assert len(a.blocks[0]) == 2
    cm.commit(a, 3)
    cm.extend(a, 1)                      # the ninth token opens a third page
    assert len(a.blocks[0]) == 3
    cm.commit(a, 1)
    b = cm.open("b")
    with pytest.raises(OutOfPages):
        cm.extend(b, 13)                 # needs 4, only 3 are free
    assert b.blocks[0] == [] and cm.num_free_pages() == 3      # nothing was taken
    assert not cm.can_extend(b, 13) and cm.can_extend(b, 12)
    assert not cm.can_extend(b, 12, reserve=[1])
    with pytest.raises(OutOfSlots):
        cm.open("c")
    with pytest.raises(CacheError, match="already open"):
        cm.open("a")
    freed = list(a.blocks[0])
    cm.close(a)
    assert cm.num_free_pages() == 6 and cm.num_free_slots == 1
    with pytest.raises(CacheError):
        cm.close(a)
    with pytest.raises(CacheError):
        cm.extend(a, 1)
    cm.extend(b, 12)                     # the pages that a gave back are used again, newest first
    assert b.blocks[0][0] == freed[-1]
    cm.check()


def test_trim_uncommitted():
    cm = CacheManager(specs_lfm2_like(), 4, 8, 2)
    a = cm.open("a")
    cm.extend(a, 6)
    cm.commit(a, 6)
    cm.extend(a, 9)
    assert len(a.blocks[0]) == 4
    cm.trim_uncommitted(a)
    assert len(a.blocks[0]) == 2 and cm.num_free_pages() == 6
    with pytest.raises(CacheError, match="more tokens than"):
        cm.commit(a, 9)


def test_window_group_gives_pages_back():
    cm = CacheManager([PagedKV(1, 8, window=6), PagedKV(1, 8)], 4, {0: 4, 1: 16}, 1)
    r = cm.open("r")
    held = []
    for step in range(40):
        cm.extend(r, 1)
        cm.commit(r, 1)
        cm.check()
        live = [p for p in r.blocks[0] if p >= 0]
        held.append(len(live))
        # every key that a query at position >= length can still see is in a live page
        first_needed = max(0, r.length - 6 + 1)
        for pos in range(first_needed, r.length):
            assert r.blocks[0][pos // 4] >= 0
        # and nothing older than one page before that is kept
        for b, page in enumerate(r.blocks[0]):
            if (b + 1) * 4 <= first_needed:
                assert page == -1
    assert max(held) <= 3                       # 6 keys never span more than 3 pages of 4
    assert len([p for p in r.blocks[1] if p >= 0]) == 10      # the full group keeps everything
    cm.close(r)
    assert cm.num_free_pages(0) == 4 and cm.num_free_pages(1) == 16


@pytest.mark.parametrize("seed", range(8))
def test_random_orders(seed):
    """Requests open, grow by random portions, and end in random order; pools of 7 to 40
    pages, sometimes with a window group.  After every action the invariants hold and the
    pages in use are exactly those the lengths need."""
    rng = random.Random(seed)
    ps = rng.choice([1, 4, 16])
    window = rng.choice([None, 5, 33])
    specs = [PagedKV(2, 16), FixedState((8, 2)), PagedKV(2, 16)]
    if window:
        specs.append(PagedKV(2, 16, window=window))
    cm = CacheManager(specs, ps, rng.randint(7, 40), rng.randint(1, 5))
    live, ended, refused = {}, 0, 0
    for step in range(600):
        action = rng.random()
        if action < 0.25 or not live:
            rid = f"q{step}"
            try:
                live[rid] = cm.open(rid)
            except OutOfSlots:
                assert cm.num_free_slots == 0
        elif action < 0.85:
            rid = rng.choice(list(live))
            rc = live[rid]
            n = rng.choice([1, 1, 1, 2, 3, 7, 20])
            before = [list(b) for b in rc.blocks]
            free_before = [cm.num_free_pages(g) for g in range(len(cm.paged_groups))]
            can = cm.can_extend(rc, n)
            try:
                cm.extend(rc, n)
                assert can
                if rng.random() < 0.1:
                    cm.trim_uncommitted(rc)          # the step failed: nothing is stored
                else:
                    cm.commit(rc, n)
            except OutOfPages:
                refused += 1
                assert not can
                assert [list(b) for b in rc.blocks] == before
                assert [cm.num_free_pages(g) for g in range(len(cm.paged_groups))] == free_before
        else:
            rid = rng.choice(list(live))
            cm.close(live.pop(rid))
            ended += 1
        cm.check()
        need = sum((rc.length + ps - 1) // ps for rc in live.values())
        assert cm.paged_groups[0].allocator.num_used == need
        slots = [rc.slot for rc in live.values()]
        assert len(set(slots)) == len(slots)
    for rc in live.values():
        cm.close(rc)
    cm.check()
    assert all(g.allocator.num_free == g.allocator.num_pages for g in cm.paged_groups)
    assert cm.num_free_slots == cm.num_slots
    assert ended > 20


def test_one_token_shortcuts_equal_the_general_calls():
    for window in (None, 6):
        a = CacheManager([PagedKV(1, 8, window=window), FixedState((4,))], 4, 12, 1)
        b = CacheManager([PagedKV(1, 8, window=window), FixedState((4,))], 4, 12, 1)
        ra, rb = a.open("x"), b.open("x")
        a.extend(ra, 3); a.commit(ra, 3)
        b.extend(rb, 3); b.commit(rb, 3)
        versions = []
        for _ in range(30):
            a.extend(ra, 1); a.commit(ra, 1)
            b.extend_one(rb); b.commit_one(rb)
            assert ra.blocks == rb.blocks and ra.length == rb.length
            a.check(); b.check()
            versions.append(rb.version)
        assert versions[-1] > versions[0]           # page changes are counted
        assert len(set(versions)) < len(versions)   # and only they


def test_a_need_describes_its_own_pools():
    """The manager serves a kind of growing state it has never heard of: one pool of latent
    vectors in float32 and one of int32 marks, two layers in a group."""
    from dataclasses import dataclass
    from typing import Optional

    import torch

    from kappai_amd.cache import PagedSpec, PoolSpec

    @dataclass(frozen=True)
    class Latent(PagedSpec):
        rank: int = 0
        window: Optional[int] = None

        def pools(self, page_size):
            return (PoolSpec("latent", (page_size, self.rank), slot_axis=0, dtype="float32"),
                    PoolSpec("mark", (2, page_size), slot_axis=1, dtype="int32"))

        def bytes_per_token(self, elem_bytes):
            return self.rank * 4 + 2 * 4

    cm = CacheManager([Latent(rank=5), PagedKV(2, 16), Latent(rank=5), FixedState((3,))], 4, 6, 2)
    assert [g.cache_ids for g in cm.paged_groups] == [[0, 2], [1]]
    assert cm.bytes_per_token(2) == 2 * (5 * 4 + 8) + 2 * 2 * 16 * 2
    cm.allocate_storage(torch.bfloat16, "cpu", poison=True)
    v = cm.view(2)
    assert v.pool("latent").shape == (7, 4, 5) and v.pool("latent").dtype == torch.float32
    assert v.pool("mark").shape == (7, 2, 4) and v.pool("mark").dtype == torch.int32
    assert torch.isnan(v.pool("latent")).all() and not v.pool("mark").any()
    kv = cm.view(1)
    assert kv.pool("k").shape == (7, 2, 4, 16) and kv.pool("v").shape == (7, 2, 16, 4)
    assert kv.pool("k").dtype == torch.bfloat16


def test_dump_gathers_a_request_out_of_its_pages():
    import torch
    cm = CacheManager([PagedKV(2, 8), FixedState((3, 2)), PagedKV(2, 8, window=5)], 4, 8, 2)
    cm.allocate_storage(torch.float32, "cpu")
    other = cm.open("other")
    cm.extend(other, 3)
    cm.commit(other, 3)
    rc = cm.open("r")
    n = 11
    cm.extend(rc, n)
    k = torch.arange(n * 2 * 8, dtype=torch.float32).reshape(n, 2, 8)
    for cid in (0, 2):
        gi = cm.view(cid).group
        for p in range(n):
            page = rc.blocks[gi][p // 4]
            cm.view(cid).pool("k")[page, :, p % 4, :] = k[p] + cid
            cm.view(cid).pool("v")[page, :, :, p % 4] = -k[p] - cid
    cm.view(1).state[rc.slot] = 7.0
    cm.commit(rc, n)                      # the window of cache 2 gives its first page back
    got = cm.export_range(rc, 0, 2, 7)
    assert torch.equal(got["k"], k[2:9]) and torch.equal(got["v"], -k[2:9])
    with pytest.raises(CacheError, match="given back"):
        cm.export_range(rc, 2, 0, 4)
    with pytest.raises(CacheError, match="not all stored"):
        cm.export_range(rc, 0, 5, 9)
    d = cm.dump(rc)
    assert d["length"] == n and d["caches"][1]["kind"] == "state"
    assert torch.equal(d["caches"][1]["state"], torch.full((3, 2), 7.0))
    assert d["caches"][0]["first_position"] == 0 and torch.equal(d["caches"][0]["k"], k)
    first = d["caches"][2]["first_position"]
    assert first == 4 and torch.equal(d["caches"][2]["v"], -k[first:] - 2)
