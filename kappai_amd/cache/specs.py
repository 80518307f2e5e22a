"""What a layer may ask of the cache manager.

A need is data: the manager reads from it how many tensors a page (or a slot) consists of, their
shapes and dtypes, and how much a token costs.  It knows nothing about what the tensors hold, so
a mixer with another kind of growing state (keys only, a latent vector per token) writes its own
``PagedSpec`` and the manager serves it unchanged.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class PoolSpec:
    """One tensor of a paged group: ``[pages, *page_shape]``.  ``slot_axis`` is the axis of
    ``page_shape`` that counts the page's token slots (its length is the page size).  ``dtype``
    None: the model's compute dtype; else the name of a torch dtype."""
    name: str
    page_shape: Tuple[int, ...]
    slot_axis: int = 0
    dtype: Optional[str] = None


class PagedSpec:
    """State that grows with the sequence, kept in pages of ``page_size`` tokens.  A subclass is
    a frozen dataclass (layers with equal specs share a group, a page id and a block table) with

    ``window``          None keeps every token; a number keeps only what the last ``window``
                        positions can still see, and pages that have fallen out of every future
                        window are given back;
    ``pools(page_size)``        the tensors of a page, as ``PoolSpec``;
    ``bytes_per_token(elem)``   bytes one token takes in one layer (``elem``: bytes of the compute
                        dtype), for sizing the pool from free memory."""
    window: Optional[int] = None

    def pools(self, page_size: int) -> Tuple[PoolSpec, ...]:
        raise NotImplementedError

    def bytes_per_token(self, elem_bytes: int) -> int:
        raise NotImplementedError


@dataclass(frozen=True)
class PagedKV(PagedSpec):
    """Keys and values of a grouped-query attention.  Keys lie ``[kv_head, slot, head_dim]`` in a
    page; values are stored transposed, ``[kv_head, head_dim, slot]``: the matrix-core attention
    kernels read eight key slots of one value column in one piece."""
    num_kv_heads: int = 1
    head_dim: int = 0
    window: Optional[int] = None

    def pools(self, page_size: int) -> Tuple[PoolSpec, ...]:
        return (PoolSpec("k", (self.num_kv_heads, page_size, self.head_dim), slot_axis=1),
                PoolSpec("v", (self.num_kv_heads, self.head_dim, page_size), slot_axis=2))

    def bytes_per_token(self, elem_bytes: int) -> int:
        return 2 * self.num_kv_heads * self.head_dim * elem_bytes


@dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size (kappai: ``kvcache_hybrid.conv_state``,
    src/kvcache.c:208-237): one slot a request, updated in place, never rewound.  A part
    that owns such state treats a segment that starts at position 0 as having no history,
    so slots are not cleared between requests (src/recipe/ops_hybrid.c:353-354)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
