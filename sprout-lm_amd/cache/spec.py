"""What a mixer asks of the cache manager."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values in pages.  window None: every earlier key stays; else only the last `window`."""

    kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size (one tensor of `shape` per request and cache slot)."""

    shape: tuple[int, ...]
    dtype: str = "float32"
