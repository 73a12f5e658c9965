"""What a mixer asks of the cache manager."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class KVNeed:
    """Keys and values per token: `num_kv_heads` heads of `head_dim`.  `window`
    None: every key is kept; W: only the last W positions are ever read, so
    pages wholly behind the window are given back.  `page_size` None: pages of
    the engine's size; P: this mixer's runs keep their keys in pages of P tokens
    (runs that ask for the same form a group with a pool of its own)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    page_size: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: a tensor of `shape` and `dtype`
    ("float32" or "bfloat16") for each request, zeroed when a request claims its slot."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
