"""What a mixer asks of the cache manager."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values in pages.  window None: every earlier key stays; else only the last `window`.
    page_tokens None: pages of the cache manager's own size; else pages of this many tokens (a divisor of the
    manager's size, which stays the unit in which prefixes are shared).
    value_dim None: values as wide as keys; else the width of a cached value where it differs from a key's
    `head_dim` (a mixer that caches a narrow rotated part beside a wide latent, say).
    dtype None: the model's cache dtype; else the name of the dtype this slot is always kept in."""

    kv_heads: int
    head_dim: int
    window: int | None = None
    page_tokens: int | None = None
    value_dim: int | None = None
    dtype: str | None = None


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size (one tensor of `shape` per request and cache slot)."""

    shape: tuple[int, ...]
    dtype: str = "float32"
