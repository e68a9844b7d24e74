"""What a mixer asks of the cache.  Schedule entries whose mixers ask for the same
thing share one group: one pool of pages and one page table (or one state table)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class KVSpec:
    """Keys and values for every token (``window`` None) or for the last ``window`` tokens.
    ``v_head_dim`` None: values have the keys' head size.  ``block``: a token only reads the keys of its own
    block of that many positions (counted from position 0), so whole blocks behind the newest token are given
    back; ``layout`` tells apart mixers that order a page's contents differently (they never share a group)."""
    n_kv_heads: int
    head_dim: int
    window: int | None = None
    v_head_dim: int | None = None
    block: int | None = None
    layout: str = "matrix"


@dataclass(frozen=True)
class StateSpec:
    """A state of fixed size for every sequence, zero when the sequence starts."""
    shape: tuple
    dtype: str = "float32"
