"""What a mixer asks of the cache.  Schedule entries whose mixers ask for the same
thing share one group: one pool of pages and one page table (or one state table)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class KVSpec:
    """Keys and values for every token (``window`` None) or for the last ``window`` tokens."""
    n_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class StateSpec:
    """A state of fixed size for every sequence, zero when the sequence starts."""
    shape: tuple
    dtype: str = "float32"
