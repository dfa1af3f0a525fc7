"""The cache a model's runs need, on the device, and the host core that hands
out its pages.

Every run of the schedule whose mixer asks for a paged need (`PagedKV`, or any class
registered as a paged kind) gets a cache layer; layers with equal needs form a group that
shares a page pool and block tables, so one page id names the same slots in every layer
of its group (as one block id does in all layers of the reference's pool,
src/kv_pool.rs:37-42).  A run that reads another run's cache shares that run's
layer and writes nothing.  Per-request needs (`FixedState`) become memory with a
row for every request slot.  How a need is laid out is its kind's business (cache/spec.py).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Optional, Sequence, Tuple, Union

import torch

from .native import HostCore
from .spec import CacheKind, CacheView, cache_kind


@dataclass
class PagedGroup:
    need: Any
    kind: CacheKind
    page_size: int
    num_pages: int
    n_layers: int
    storage: Any
    dtype: torch.dtype

    def bytes_per_token(self) -> int:
        return self.n_layers * self.kind.bytes_per_token(self.need, self.dtype)


def _group_runs(needs: Sequence[Tuple[object, Optional[int]]]):
    """(the distinct paged needs, layers in each, (group, layer) of every run or None, the runs with per-request needs)."""
    group_needs: List[Any] = []
    layers_in_group: List[int] = []
    layer_of_run: List[Optional[Tuple[int, int]]] = []
    per_request: List[int] = []
    for i, (need, cache_of) in enumerate(needs):
        paged = need is not None and cache_kind(need).paged
        if not paged:
            if cache_of is not None:
                raise ValueError(f"run {i} reads the cache of run {cache_of} but its mixer keeps no paged cache")
            layer_of_run.append(None)
            if need is not None:
                per_request.append(i)
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
    return group_needs, layers_in_group, layer_of_run, per_request


class CacheManager:
    def __init__(self, needs: Sequence[Tuple[object, Optional[int]]], dtype: torch.dtype, device,
                 page_size: int, num_pages: Union[int, Sequence[int]], max_requests: int,
                 token_budget: int = 2048, max_chunk: int = 0, max_positions: int = 1 << 30):
        """`needs[i]` = (what run i's mixer asks for, index of the run whose cache it reads or None)."""
        self.dtype, self.device = dtype, device
        self.page_size, self.max_requests = page_size, max_requests
        group_needs, layers_in_group, layer_of_run, per_request = _group_runs(needs)
        pages = [int(num_pages)] * len(group_needs) if isinstance(num_pages, int) else [int(n) for n in num_pages]
        if len(pages) != len(group_needs):
            raise ValueError(f"num_pages names {len(pages)} groups, the model has {len(group_needs)}")
        self.groups: List[PagedGroup] = []
        for need, n_layers, n_pages in zip(group_needs, layers_in_group, pages):
            kind = cache_kind(need)
            self.groups.append(PagedGroup(need, kind, page_size, n_pages, n_layers,
                                          kind.allocate_pages(need, n_layers, n_pages, page_size, dtype, device), dtype))
        self.views: List[CacheView] = []
        self._per_request: List[Tuple[CacheKind, Any, Any]] = []      # (kind, need, storage) of the runs with such needs
        for i, (need, cache_of) in enumerate(needs):
            if need is None:
                self.views.append(CacheView("none"))
            elif layer_of_run[i] is not None:
                g, layer = layer_of_run[i]
                grp = self.groups[g]
                self.views.append(grp.kind.page_view(grp.storage, need, layer, g, page_size, grp.num_pages, cache_of is None))
            else:
                kind = cache_kind(need)
                storage = kind.allocate_slots(need, max_requests, device)
                self._per_request.append((kind, need, storage))
                self.views.append(kind.slot_view(storage, need))
        self.core = HostCore([(page_size, g.num_pages, g.kind.window(g.need)) for g in self.groups], max_requests,
                             token_budget, max_chunk, max_positions)

    @staticmethod
    def pages_that_fit(needs: Sequence[Tuple[object, Optional[int]]], dtype: torch.dtype, page_size: int, free_bytes: int,
                       fraction: float, max_requests: int, max_seq_len: int, max_step_tokens: int = 0) -> List[int]:
        """Pages for each group such that all of them take `fraction` of `free_bytes` less what the per-request
        needs take (src/kv_pool.rs:26-35 sizes its pool the same way, from RAM).  No group gets more than
        `max_requests` requests could ever hold: `max_seq_len` tokens each, or, in a group with a window, the
        window and the `max_step_tokens` tokens of a step's portion; what such a group does not need goes to the
        others."""
        group_needs, layers_in_group, _, per_request = _group_runs(needs)
        if not group_needs:
            return []
        fixed = sum(cache_kind(needs[i][0]).bytes_per_request(needs[i][0]) for i in per_request) * max_requests
        budget = int(max(free_bytes - fixed, 0) * fraction)
        step = min(max_step_tokens or max_seq_len, max_seq_len)
        caps, costs = [], []
        for need, n_layers in zip(group_needs, layers_in_group):
            kind = cache_kind(need)
            held = max_seq_len
            if kind.window(need) > 0:
                # a page's worth more than the span: the span starts anywhere in a page
                held = min(held, kind.window(need) + step + page_size)
            caps.append(max_requests * -(-held // page_size))
            costs.append(n_layers * kind.bytes_per_token(need, dtype) * page_size)
        lo, hi = 1, max(caps)          # the most pages P with sum(cost * min(cap, P)) within the budget, at least one
        while lo < hi:
            mid = (lo + hi + 1) // 2
            if sum(c * min(cap, mid) for c, cap in zip(costs, caps)) <= budget:
                lo = mid
            else:
                hi = mid - 1
        return [min(cap, lo) for cap in caps]

    def bytes_per_token(self) -> int:
        return sum(g.bytes_per_token() for g in self.groups)

    @property
    def state_tensors(self) -> List[Any]:
        """What the per-request needs were given, in the order of their runs."""
        return [storage for _, _, storage in self._per_request]

    def reset_state(self, slots: Sequence[int]) -> None:
        """Per-request memory starts afresh when a request starts (or starts again) at position 0."""
        if self._per_request and len(slots):
            idx = torch.as_tensor(list(slots), dtype=torch.long, device=self.device)
            for kind, need, storage in self._per_request:
                kind.reset_slots(storage, need, idx)
