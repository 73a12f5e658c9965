"""What a mixer asks of the cache manager."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class KVNeed:
    """Keys and values per token: `num_kv_heads` heads of `head_dim`.  `window`
    None: every key is kept; W: only the last W positions are ever read, so
    pages wholly behind the window are given back."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: a tensor of `shape` and `dtype`
    ("float32" or "bfloat16") for each request, zeroed when a request claims its slot."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
