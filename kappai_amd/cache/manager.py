"""The cache manager: pages of keys and values with a block table per request, and slots
for per-request state of fixed size.

kappai gives every session one contiguous K/V allocation of the full context and a conv
state beside it (src/kvcache.c:166-314).  Here the layers that own a cache are put into
groups by what they need: each group of paged layers has a page pool of its own (one
page id addresses the same page in every layer of the group) and a block table per
request; each group of fixed-state layers has an array of slots.  Pages return to the
pool when a request ends or when a window has passed them, and are handed out again
(most recently freed first, so that reuse happens early).

The bookkeeping is plain Python and needs no GPU; only ``allocate_storage`` touches the
device.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Union

import numpy as np
import torch

from .specs import FixedState, PagedSpec


class CacheError(RuntimeError):
    """Misuse of the cache manager (a bug in the caller)."""


class OutOfPages(RuntimeError):
    """A group's pool cannot hold the tokens asked for.  Nothing was allocated."""


class OutOfSlots(RuntimeError):
    """Every state slot is taken.  Nothing was allocated."""


class PageAllocator:
    """Free list of page ids with an owner per page: a page is never lost, never held
    twice and never freed twice."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise CacheError("a pool cannot have a negative number of pages")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._owner: List[Optional[Hashable]] = [None] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def take(self, owner: Hashable) -> int:
        if owner is None:
            raise CacheError("a page needs an owner")
        if not self._free:
            raise OutOfPages("the page pool is empty")
        page = self._free.pop()
        if self._owner[page] is not None:
            raise CacheError(f"page {page} was on the free list while owned by "
                             f"{self._owner[page]!r}")
        self._owner[page] = owner
        return page

    def give_back(self, page: int, owner: Hashable) -> None:
        if not 0 <= page < self.num_pages:
            raise CacheError(f"page {page} does not exist")
        if self._owner[page] is None:
            raise CacheError(f"page {page} is freed twice")
        if self._owner[page] != owner:
            raise CacheError(f"page {page} belongs to {self._owner[page]!r}, not to {owner!r}")
        self._owner[page] = None
        self._free.append(page)

    def owner_of(self, page: int):
        return self._owner[page]

    def check(self) -> None:
        """Invariant: free list and owners describe the same partition of the pool."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise CacheError("a page is on the free list twice")
        for p in range(self.num_pages):
            if (p in free) == (self._owner[p] is not None):
                raise CacheError(f"page {p} is {'free and owned' if p in free else 'lost'}")


@dataclass
class PagedGroup:
    spec: PagedSpec
    cache_ids: List[int]
    allocator: PageAllocator
    # cache id -> {pool name: tensor [pages + 1, *page_shape]}, as the spec's pools() names them
    pools: Dict[int, Dict[str, torch.Tensor]] = field(default_factory=dict)


@dataclass
class StateGroup:
    spec: FixedState
    cache_ids: List[int]
    states: Dict[int, torch.Tensor] = field(default_factory=dict)    # cache id -> [slots, *shape]


@dataclass
class PagedLayerView:
    """What a paged layer sees: its pools by the names its spec gave them (empty before
    ``allocate_storage``) and the index of its group's block tables."""
    pools: Dict[str, torch.Tensor]
    group: int
    spec: PagedSpec
    page_size: int

    def pool(self, name: str) -> Optional[torch.Tensor]:
        return self.pools.get(name)


@dataclass
class StateLayerView:
    state: Optional[torch.Tensor]
    group: int
    spec: FixedState


class RequestCache:
    """Everything one live request holds: a slot, and per paged group its block table.
    ``length`` counts the tokens whose keys are stored."""

    def __init__(self, request_id: Hashable, slot: int, n_paged_groups: int):
        self.request_id = request_id
        self.slot = slot
        self.length = 0
        self.blocks: List[List[int]] = [[] for _ in range(n_paged_groups)]  # -1 = given back
        self.closed = False
        self.version = 0        # counts changes of `blocks`, for callers that mirror them
        self._arrays = [(-1, None)] * n_paged_groups      # (version, blocks[g] as int32 array)

    def block_array(self, group: int):
        """``blocks[group]`` as an int32 array, made anew only when the list has changed (a page
        is taken every ``page_size`` tokens, so the step function copies the same array into its
        tables for many steps in a row)."""
        version, array = self._arrays[group]
        if version != self.version:
            array = np.asarray(self.blocks[group], dtype=np.int32)
            self._arrays[group] = (self.version, array)
        return array

    def __repr__(self):
        return f"RequestCache({self.request_id!r}, slot={self.slot}, length={self.length})"


Spec = Union[PagedSpec, FixedState, None]


class CacheManager:
    def __init__(self, cache_specs: Sequence[Spec], page_size: int,
                 num_pages: Union[int, Dict[int, int]], num_slots: int):
        """``cache_specs[i]`` is what cache ``i`` needs (None: nothing).  ``num_pages`` is the
        size of every paged group's pool, or a dictionary from group index to size."""
        if page_size < 1:
            raise CacheError("page_size must be at least 1")
        if num_slots < 1:
            raise CacheError("at least one slot is needed")
        self.page_size = page_size
        self.num_slots = num_slots
        self.cache_specs = list(cache_specs)
        self.paged_groups: List[PagedGroup] = []
        self.state_groups: List[StateGroup] = []
        self._where: Dict[int, tuple] = {}
        for cid, spec in enumerate(self.cache_specs):
            if spec is None:
                continue
            if isinstance(spec, PagedSpec):
                groups, kind = self.paged_groups, "paged"
            elif isinstance(spec, FixedState):
                groups, kind = self.state_groups, "state"
            else:
                raise CacheError(f"cache {cid}: unknown cache need {spec!r}")
            for gi, g in enumerate(groups):
                if g.spec == spec:
                    g.cache_ids.append(cid)
                    self._where[cid] = (kind, gi)
                    break
            else:
                gi = len(groups)
                if kind == "paged":
                    n = num_pages[gi] if isinstance(num_pages, dict) else num_pages
                    groups.append(PagedGroup(spec, [cid], PageAllocator(int(n))))
                else:
                    groups.append(StateGroup(spec, [cid]))
                self._where[cid] = (kind, gi)
        self._free_slots: List[int] = list(range(num_slots - 1, -1, -1))
        self._live: Dict[Hashable, RequestCache] = {}
        self._has_windows = any(g.spec.window for g in self.paged_groups)
        self.device = None
        self.dtype = None

    # -- device storage -------------------------------------------------------------------
    def allocate_storage(self, dtype: torch.dtype, device, poison: bool = False) -> None:
        """Create, for every layer of a paged group, the tensors its spec names
        (``[pages + 1, *page_shape]`` each), and the slot arrays.  ``poison`` fills them with NaN
        so that a read of something nobody wrote shows."""
        self.device, self.dtype = device, dtype
        for g in self.paged_groups:
            n = g.allocator.num_pages + 1          # the last page is scratch (see scratch_page)
            for cid in g.cache_ids:
                made = {}
                for pool in g.spec.pools(self.page_size):
                    pdt = dtype if pool.dtype is None else getattr(torch, pool.dtype)
                    t = torch.empty((n, *pool.page_shape), dtype=pdt, device=device)
                    if poison and pdt.is_floating_point:
                        t.fill_(float("nan"))
                    else:
                        t.zero_()
                    made[pool.name] = t
                g.pools[cid] = made
        for g in self.state_groups:
            sdt = getattr(torch, g.spec.dtype)
            for cid in g.cache_ids:
                t = torch.zeros((self.num_slots + 1, *g.spec.shape), dtype=sdt, device=device)
                if poison:
                    t.fill_(float("nan"))
                g.states[cid] = t

    def scratch_page(self, group: int) -> int:
        """A page beyond the allocator's reach that no request ever reads: rows of a warm-up
        run are stored there."""
        return self.paged_groups[group].allocator.num_pages

    @property
    def scratch_slot(self) -> int:
        """A state slot beyond the allocator's reach, for warm-up runs."""
        return self.num_slots

    def bytes_per_token(self, dtype_bytes: int) -> int:
        """Bytes that one token takes over all paged layers (kappai:
        model_kv_cache_bytes_quant, src/memory.c:292)."""
        return sum(g.spec.bytes_per_token(dtype_bytes) * len(g.cache_ids)
                   for g in self.paged_groups)

    def view(self, cache_id: int):
        if cache_id not in self._where:
            raise CacheError(f"cache {cache_id} was declared to need nothing")
        kind, gi = self._where[cache_id]
        if kind == "paged":
            g = self.paged_groups[gi]
            return PagedLayerView(g.pools.get(cache_id, {}), gi, g.spec, self.page_size)
        g = self.state_groups[gi]
        return StateLayerView(g.states.get(cache_id), gi, g.spec)

    # -- looking into a request's cache ------------------------------------------------------
    def export_range(self, rc: RequestCache, cache_id: int, pos_start: int = 0,
                     n_rows: Optional[int] = None) -> Dict[str, torch.Tensor]:
        """What the paged cache ``cache_id`` holds for positions ``pos_start .. pos_start +
        n_rows - 1`` of the request, gathered out of its pages: ``{pool name: [n_rows, *rest]}``
        with the token first and the other axes of a page in their order (keys
        ``[n, kv_heads, head_dim]``, values the same, whatever the page's layout).  For looking
        at a request when a page goes wrong (kappai: kvcache_export_range, src/kvcache.c:887-901).
        A position whose page a window has given back is an error."""
        self._check_live(rc)
        kind, gi = self._where.get(cache_id, (None, None))
        if kind != "paged":
            raise CacheError(f"cache {cache_id} is not a paged cache")
        g = self.paged_groups[gi]
        if cache_id not in g.pools:
            raise CacheError("allocate_storage has not been called")
        n_rows = rc.length - pos_start if n_rows is None else n_rows
        if pos_start < 0 or n_rows < 0 or pos_start + n_rows > rc.length:
            raise CacheError(f"{rc}: positions {pos_start}..{pos_start + n_rows - 1} are not all "
                             "stored")
        pos = torch.arange(pos_start, pos_start + n_rows)
        blocks = torch.tensor(rc.blocks[gi] or [0], dtype=torch.long)
        pages = blocks[pos // self.page_size] if n_rows else pos
        if n_rows and int(pages.min()) < 0:
            gone = int(pos[pages < 0][0])
            raise CacheError(f"{rc}: position {gone} of cache {cache_id} lies in a page that its "
                             f"window ({g.spec.window}) has given back")
        slots = pos % self.page_size
        out = {}
        for pool in g.spec.pools(self.page_size):
            t = g.pools[cache_id][pool.name]
            moved = t.movedim(1 + pool.slot_axis, 1)            # [pages, slot, *rest]
            out[pool.name] = moved[pages.to(t.device), slots.to(t.device)].clone()
        return out

    def export_state(self, rc: RequestCache, cache_id: int) -> torch.Tensor:
        """A copy of the request's slot of the fixed-size state ``cache_id`` (kappai:
        kvcache_export_state, src/kvcache.c:924-945)."""
        self._check_live(rc)
        kind, gi = self._where.get(cache_id, (None, None))
        if kind != "state":
            raise CacheError(f"cache {cache_id} is not a fixed-size state")
        g = self.state_groups[gi]
        if cache_id not in g.states:
            raise CacheError("allocate_storage has not been called")
        return g.states[cache_id][rc.slot].clone()

    def dump(self, rc: RequestCache) -> dict:
        """Everything the request holds, for debugging: its length, slot and block tables, and
        per cache id what ``export_range`` (the positions still kept) or ``export_state`` gives."""
        self._check_live(rc)
        out = {"request": rc.request_id, "length": rc.length, "slot": rc.slot,
               "blocks": [list(b) for b in rc.blocks], "caches": {}}
        for cid, (kind, gi) in sorted(self._where.items()):
            if kind == "state":
                out["caches"][cid] = {"kind": "state", "state": self.export_state(rc, cid)}
                continue
            first = next((i for i, b in enumerate(rc.blocks[gi]) if b >= 0), 0) * self.page_size
            first = min(first, rc.length)
            out["caches"][cid] = {"kind": "paged", "first_position": first,
                                  **self.export_range(rc, cid, first, rc.length - first)}
        return out

    # -- requests -------------------------------------------------------------------------
    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def num_free_pages(self, group: int = 0) -> int:
        return self.paged_groups[group].allocator.num_free

    def live_requests(self):
        return list(self._live.values())

    def open(self, request_id: Hashable) -> RequestCache:
        if request_id in self._live:
            raise CacheError(f"request {request_id!r} is already open")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.num_slots} state slots are taken")
        rc = RequestCache(request_id, self._free_slots.pop(), len(self.paged_groups))
        self._live[request_id] = rc
        return rc

    def _blocks_for(self, n_tokens: int) -> int:
        return (n_tokens + self.page_size - 1) // self.page_size

    def pages_needed(self, rc: RequestCache, n_new: int) -> List[int]:
        """Per paged group, the pages that ``n_new`` more tokens would take."""
        want = self._blocks_for(rc.length + n_new)
        return [max(0, want - len(b)) for b in rc.blocks]

    def can_extend(self, rc: RequestCache, n_new: int, reserve: Optional[List[int]] = None) -> bool:
        """True if ``extend`` would succeed; ``reserve`` counts pages per group that other
        entries of the same step will take first."""
        need = self.pages_needed(rc, n_new)
        for gi, g in enumerate(self.paged_groups):
            if need[gi] + (reserve[gi] if reserve else 0) > g.allocator.num_free:
                return False
        return True

    def can_extend_all(self, caches: Sequence[RequestCache], n_new: int) -> bool:
        """True if every one of ``caches`` can grow by ``n_new`` tokens at the same time (pages
        that a window would give back meanwhile are not counted on)."""
        total = [0] * len(self.paged_groups)
        for rc in caches:
            for gi, need in enumerate(self.pages_needed(rc, n_new)):
                total[gi] += need
        return all(total[gi] <= g.allocator.num_free for gi, g in enumerate(self.paged_groups))

    def extend(self, rc: RequestCache, n_new: int) -> None:
        """Make room for tokens ``length .. length + n_new - 1`` in every paged group.
        Either every group gets its pages or nothing changes."""
        self._check_live(rc)
        if n_new < 1:
            raise CacheError("extend needs at least one token")
        need = self.pages_needed(rc, n_new)
        for gi, g in enumerate(self.paged_groups):
            if need[gi] > g.allocator.num_free:
                raise OutOfPages(
                    f"request {rc.request_id!r} needs {need[gi]} more pages of group {gi} "
                    f"(window={g.spec.window}) for {n_new} tokens at length {rc.length}; "
                    f"{g.allocator.num_free} of {g.allocator.num_pages} are free")
        for gi, g in enumerate(self.paged_groups):
            for _ in range(need[gi]):
                rc.blocks[gi].append(g.allocator.take(rc.request_id))
        if any(need):
            rc.version += 1

    def extend_one(self, rc: RequestCache) -> None:
        """``extend(rc, 1)`` for the common case of a decoded token: nothing to do unless the
        token opens a new page."""
        if rc.length % self.page_size == 0 or any(
                len(b) * self.page_size <= rc.length for b in rc.blocks):
            self.extend(rc, 1)
        elif rc.closed:
            raise CacheError(f"{rc} is not an open request of this cache")

    def commit_one(self, rc: RequestCache) -> None:
        """``commit(rc, 1)``; without window groups only the length changes."""
        if self._has_windows:
            self.commit(rc, 1)
        else:
            rc.length += 1

    def commit(self, rc: RequestCache, n_new: int) -> None:
        """The step has stored ``n_new`` tokens.  Pages that no later position can see
        through its window go back to the pool."""
        self._check_live(rc)
        rc.length += n_new
        if self._blocks_for(rc.length) > min((len(b) for b in rc.blocks), default=10 ** 18):
            raise CacheError(f"{rc}: committed more tokens than were made room for")
        for gi, g in enumerate(self.paged_groups):
            w = g.spec.window
            if not w:
                continue
            first_needed = rc.length - w + 1      # oldest key a query at position >= length sees
            b = 0
            while (b + 1) * self.page_size <= first_needed and b < len(rc.blocks[gi]):
                if rc.blocks[gi][b] >= 0:
                    g.allocator.give_back(rc.blocks[gi][b], rc.request_id)
                    rc.blocks[gi][b] = -1
                    rc.version += 1
                b += 1

    def trim_uncommitted(self, rc: RequestCache) -> None:
        """Give back pages that ``extend`` took for tokens that were never committed."""
        keep = self._blocks_for(rc.length)
        for gi, g in enumerate(self.paged_groups):
            while len(rc.blocks[gi]) > keep:
                page = rc.blocks[gi].pop()
                rc.version += 1
                if page >= 0:
                    g.allocator.give_back(page, rc.request_id)

    def close(self, rc: RequestCache) -> None:
        """The request has ended: all its pages and its slot return to the free lists."""
        self._check_live(rc)
        for gi, g in enumerate(self.paged_groups):
            for page in rc.blocks[gi]:
                if page >= 0:
                    g.allocator.give_back(page, rc.request_id)
            rc.blocks[gi] = []
        rc.version += 1
        self._free_slots.append(rc.slot)
        del self._live[rc.request_id]
        rc.closed = True

    def _check_live(self, rc: RequestCache) -> None:
        if rc.closed or self._live.get(rc.request_id) is not rc:
            raise CacheError(f"{rc} is not an open request of this cache")

    def check(self) -> None:
        """Invariants over everything held: used pages = pages in block tables, no page in
        two tables, slots distinct, free + used = total."""
        for gi, g in enumerate(self.paged_groups):
            g.allocator.check()
            seen = {}
            for rc in self._live.values():
                if rc.block_array(gi).tolist() != rc.blocks[gi]:
                    raise CacheError(f"{rc.request_id!r}: the array form of its block table of "
                                     f"group {gi} is out of date")
                for page in rc.blocks[gi]:
                    if page < 0:
                        continue
                    if page in seen:
                        raise CacheError(f"page {page} of group {gi} is in the tables of "
                                         f"{seen[page]!r} and {rc.request_id!r}")
                    if g.allocator.owner_of(page) != rc.request_id:
                        raise CacheError(f"page {page} of group {gi} is in the table of "
                                         f"{rc.request_id!r} but owned by "
                                         f"{g.allocator.owner_of(page)!r}")
                    seen[page] = rc.request_id
            if len(seen) != g.allocator.num_used:
                raise CacheError(f"group {gi}: {g.allocator.num_used} pages are taken but "
                                 f"{len(seen)} are in block tables")
        slots = [rc.slot for rc in self._live.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise CacheError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.num_slots:
            raise CacheError("a state slot was lost")
