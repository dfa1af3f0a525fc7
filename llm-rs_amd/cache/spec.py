"""What a mixer tells the cache manager about the memory it needs per request, and how each
kind of need becomes memory.

A need is a small frozen value (`PagedKV`, `FixedState`, or one of a class that somebody
registered); the `CacheKind` registered for its class says what it costs and how it is laid out.
There are two families.  A *paged* kind holds something for every token of a request: runs
of the schedule with equal needs share a pool of pages and one block table per request, and a
window lets pages that no later query can see go back.  A *per-request* kind holds something
of fixed size for every request slot.  The cache manager, the engine's sizing of the pool and
the step function know the two families, never a particular kind.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch


@dataclass(frozen=True)
class PagedKV:
    """Keys and values in pages; `window` > 0 means only that many of the latest
    keys stay visible, so older pages can go back to the pool.  `value_dim`: the width of a
    value when it is not the width of a key (0: the same)."""
    kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: int = 0

    @property
    def v_dim(self) -> int:
        return self.value_dim or self.head_dim


@dataclass(frozen=True)
class FixedState:
    """State of a fixed size per request, kept in the request's slot."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class CacheView:
    """What one run's mixer sees of the cache."""
    kind: str                       # "paged", "state", "none", or what another kind calls itself
    group: int = -1                 # index into the step's slot maps and block tables (paged kinds)
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    page_size: int = 0
    num_pages: int = 0
    writes: bool = True
    state: Optional[torch.Tensor] = None   # [max_requests, *shape]
    data: Any = None                # whatever a kind registered from outside hands its mixer


class CacheKind:
    """How needs of one class become memory.  `paged` says which family the kind belongs to."""

    paged = False

    # -- paged kinds ---------------------------------------------------------------
    def window(self, need) -> int:
        """Tokens that stay visible (0: all): pages that lie wholly before them go back to the pool."""
        return 0

    def bytes_per_token(self, need, dtype: torch.dtype) -> int:
        """Bytes one token takes in one layer of this need."""
        raise NotImplementedError

    def allocate_pages(self, need, n_layers: int, num_pages: int, page_size: int, dtype: torch.dtype, device) -> Any:
        """The memory of a group: `n_layers` layers of `num_pages` pages of `page_size` tokens."""
        raise NotImplementedError

    def page_view(self, storage, need, layer: int, group: int, page_size: int, num_pages: int, writes: bool) -> CacheView:
        """What the mixer of the run that owns (or reads) layer `layer` of the group gets."""
        raise NotImplementedError

    # -- per-request kinds -----------------------------------------------------------
    def bytes_per_request(self, need) -> int:
        raise NotImplementedError

    def allocate_slots(self, need, max_requests: int, device) -> Any:
        raise NotImplementedError

    def slot_view(self, storage, need) -> CacheView:
        raise NotImplementedError

    def reset_slots(self, storage, need, slots: torch.Tensor) -> None:
        """A request starts (or starts again) at position 0 in each of `slots` (int64, on the device)."""
        raise NotImplementedError


class _PagedKVKind(CacheKind):
    """keys [layer][page][kv_head][slot][head_dim], values [layer][page][kv_head][value_dim][slot]
    (values transposed, so that the index the second product contracts is contiguous: csrc/hip/cache_layout.h)."""
    paged = True

    def window(self, need):
        return need.window

    def bytes_per_token(self, need, dtype):
        return need.kv_heads * (need.head_dim + need.v_dim) * dtype.itemsize

    def allocate_pages(self, need, n_layers, num_pages, page_size, dtype, device):
        k = torch.zeros((n_layers, num_pages, need.kv_heads, page_size, need.head_dim), dtype=dtype, device=device)
        v = torch.zeros((n_layers, num_pages, need.kv_heads, need.v_dim, page_size), dtype=dtype, device=device)
        return k, v

    def page_view(self, storage, need, layer, group, page_size, num_pages, writes):
        return CacheView("paged", group, storage[0][layer], storage[1][layer], page_size, num_pages, writes=writes)


class _FixedStateKind(CacheKind):
    def bytes_per_request(self, need):
        n = need.dtype.itemsize
        for s in need.shape:
            n *= int(s)
        return n

    def allocate_slots(self, need, max_requests, device):
        return torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)

    def slot_view(self, storage, need):
        return CacheView("state", state=storage)

    def reset_slots(self, storage, need, slots):
        storage.index_fill_(0, slots, 0)


_KINDS: Dict[type, CacheKind] = {}


def register_cache_kind(need_class: type, kind: CacheKind) -> None:
    """Needs of class `need_class` (hashable values that compare equal when they can share memory) are
    served by `kind` from now on."""
    _KINDS[need_class] = kind


def cache_kind(need) -> CacheKind:
    kind = _KINDS.get(type(need))
    if kind is None:
        raise TypeError(f"a mixer's cache need must be None or of a registered class "
                        f"({', '.join(sorted(c.__name__ for c in _KINDS))}), got {need!r}")
    return kind


register_cache_kind(PagedKV, _PagedKVKind())
register_cache_kind(FixedState, _FixedStateKind())
