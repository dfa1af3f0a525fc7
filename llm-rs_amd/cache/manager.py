"""The cache a model's runs need, on the device, and the host core that hands
out its pages.

Every run of the schedule whose mixer asks for `PagedKV` gets a cache layer;
layers with equal needs (kv heads, head size, window) form a group that shares a
page pool and block tables, so one page id names the same slots in every layer
of its group (as one block id does in all layers of the reference's pool,
src/kv_pool.rs:37-42).  A run that reads another run's cache shares that run's
layer and writes nothing.  `FixedState` needs become one tensor per run with a
row for every request slot.

Layout of a group (csrc/hip/cache_layout.h):
  keys   [layer][page][kv_head][slot][head_dim]
  values [layer][page][kv_head][head_dim][slot]
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple, Union

import torch

from .native import HostCore
from .spec import FixedState, PagedKV


@dataclass
class CacheView:
    """What one run's mixer sees of the cache."""
    kind: str                       # "paged", "state" or "none"
    group: int = -1                 # index into the step's slot maps and block tables
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    page_size: int = 0
    num_pages: int = 0
    writes: bool = True
    state: Optional[torch.Tensor] = None   # [max_requests, *shape]


@dataclass
class PagedGroup:
    need: PagedKV
    page_size: int
    num_pages: int
    n_layers: int
    k: torch.Tensor
    v: torch.Tensor

    def bytes_per_token(self) -> int:
        return 2 * self.n_layers * self.need.kv_heads * self.need.head_dim * self.k.element_size()


class CacheManager:
    def __init__(self, needs: Sequence[Tuple[object, Optional[int]]], dtype: torch.dtype, device,
                 page_size: int, num_pages: Union[int, Sequence[int]], max_requests: int,
                 token_budget: int = 2048, max_chunk: int = 0, max_positions: int = 1 << 30):
        """`needs[i]` = (what run i's mixer asks for, index of the run whose cache it reads or None)."""
        self.dtype, self.device = dtype, device
        self.page_size, self.max_requests = page_size, max_requests
        group_needs: List[PagedKV] = []
        layer_of_run: List[Optional[Tuple[int, int]]] = []
        layers_in_group: List[int] = []
        for i, (need, cache_of) in enumerate(needs):
            if not isinstance(need, PagedKV):
                if cache_of is not None:
                    raise ValueError(f"run {i} reads the cache of run {cache_of} but its mixer keeps no paged cache")
                layer_of_run.append(None)
                continue
            if cache_of is not None:
                src_need = needs[cache_of][0]
                if src_need != need or layer_of_run[cache_of] is None:
                    raise ValueError(f"run {i} reads the cache of run {cache_of}, whose cache has other sizes: {src_need} vs {need}")
                layer_of_run.append(layer_of_run[cache_of])
                continue
            if need not in group_needs:
                group_needs.append(need)
                layers_in_group.append(0)
            g = group_needs.index(need)
            layer_of_run.append((g, layers_in_group[g]))
            layers_in_group[g] += 1
        pages = [int(num_pages)] * len(group_needs) if isinstance(num_pages, int) else [int(n) for n in num_pages]
        if len(pages) != len(group_needs):
            raise ValueError(f"num_pages names {len(pages)} groups, the model has {len(group_needs)}")
        self.groups: List[PagedGroup] = []
        for need, n_layers, n_pages in zip(group_needs, layers_in_group, pages):
            shape_k = (n_layers, n_pages, need.kv_heads, page_size, need.head_dim)
            shape_v = (n_layers, n_pages, need.kv_heads, need.head_dim, page_size)
            self.groups.append(PagedGroup(need, page_size, n_pages, n_layers,
                                          torch.zeros(shape_k, dtype=dtype, device=device),
                                          torch.zeros(shape_v, dtype=dtype, device=device)))
        self.views: List[CacheView] = []
        self.state_tensors: List[torch.Tensor] = []
        for i, (need, cache_of) in enumerate(needs):
            if isinstance(need, PagedKV):
                g, layer = layer_of_run[i]
                grp = self.groups[g]
                self.views.append(CacheView("paged", g, grp.k[layer], grp.v[layer], page_size, grp.num_pages,
                                            writes=cache_of is None))
            elif isinstance(need, FixedState):
                state = torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)
                self.state_tensors.append(state)
                self.views.append(CacheView("state", state=state))
            elif need is None:
                self.views.append(CacheView("none"))
            else:
                raise TypeError(f"run {i}: a mixer's cache need must be PagedKV, FixedState or None, got {need!r}")
        self.core = HostCore([(page_size, g.num_pages, g.need.window) for g in self.groups], max_requests,
                             token_budget, max_chunk, max_positions)

    def bytes_per_token(self) -> int:
        return sum(g.bytes_per_token() for g in self.groups)

    def reset_state(self, slots: Sequence[int]) -> None:
        """Fixed-size state starts from zero when a request starts (or starts again) at position 0."""
        if self.state_tensors and len(slots):
            idx = torch.as_tensor(list(slots), dtype=torch.long, device=self.device)
            for s in self.state_tensors:
                s.index_fill_(0, idx, 0)
