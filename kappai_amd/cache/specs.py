"""What a layer may ask of the cache manager."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class PagedKV:
    """Keys and values that grow with the sequence, kept in pages.  ``window`` None keeps
    every key; a number keeps only what the last ``window`` positions can still see, and
    pages that have fallen out of every future window are given back."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size (kappai: ``kvcache_hybrid.conv_state``,
    src/kvcache.c:208-237): one slot a request, updated in place, never rewound.  A part
    that owns such state treats a segment that starts at position 0 as having no history,
    so slots are not cleared between requests (src/recipe/ops_hybrid.c:353-354)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
