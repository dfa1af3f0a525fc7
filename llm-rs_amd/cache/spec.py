"""What a mixer tells the cache manager about the memory it needs per request."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch


@dataclass(frozen=True)
class PagedKV:
    """Keys and values in pages; `window` > 0 means only that many of the latest
    keys stay visible, so older pages can go back to the pool."""
    kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class FixedState:
    """State of a fixed size per request, kept in the request's slot."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
