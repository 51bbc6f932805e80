"""What a mixer asks of the cache manager for one cache entry."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every token, in pages.  window > 0: only the last `window` positions
    before (and including) a query are ever read, so older pages can be given back."""
    num_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class FixedState:
    """State of fixed size per request (one row of a pool per request); row 0 is all zeros and
    is what a request starts from."""
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None  # None: float32
