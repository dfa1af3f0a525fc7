"""The cache manager on the host: pages conserved, never held twice or freed
twice, all-or-nothing growth, windows give pages back, pages are used again,
under random orders of requests.  Reference behaviours: pop order 0,1,2...
(src/kv_pool.rs:43), all-or-nothing ensure_blocks (src/kv_pool.rs:83-95), stable
slots (src/serve/engine.rs:69-92)."""
import random

import numpy as np
import pytest

from llm_rs_amd.cache import CoreError, HostCore


def held_pages(core, slots, g=0):
    pages = []
    for s in slots:
        pages += [p for p in core.table(s, g) if p >= 0]
    return pages


def check_invariants(core, slots):
    for g in range(core.n_groups):
        pages = held_pages(core, slots, g)
        assert len(pages) == len(set(pages)), "a page is held twice"
        assert all(0 <= p < core.pages_total(g) for p in pages)
        assert core.pages_free(g) + len(pages) == core.pages_total(g), "a page was lost"
        for s in slots:
            assert core.pages_held(s, g) == len([p for p in core.table(s, g) if p >= 0])


def test_pages_come_in_order_and_come_back():
    core = HostCore([(4, 8, 0)], max_requests=4)
    a = core.acquire_slot()
    assert core.ensure(a, 0, 9) and core.table(a) == [0, 1, 2]          # ceil(9/4) pages, popped 0,1,2
    b = core.acquire_slot()
    assert core.ensure(b, 0, 4) and core.table(b) == [3]
    assert core.ensure(a, 9, 3) and core.table(a) == [0, 1, 2]          # 12 tokens still fit 3 pages
    assert core.ensure(a, 12, 1) and core.table(a) == [0, 1, 2, 4]
    core.release_slot(b)
    c = core.acquire_slot()
    assert c == b, "a freed slot is the next one handed out"
    assert core.ensure(c, 0, 1) and core.table(c) == [3], "a freed page is used again, last freed first"
    check_invariants(core, [a, c])


def test_growth_is_all_or_nothing():
    core = HostCore([(4, 4, 0)], max_requests=2)
    a, b = core.acquire_slot(), core.acquire_slot()
    assert core.ensure(a, 0, 8)
    assert not core.ensure(b, 0, 12), "3 pages wanted, 2 free"
    assert core.table(b) == [] and core.pages_free() == 2, "a failed request takes nothing"
    assert core.ensure(b, 0, 8) and core.pages_free() == 0
    assert not core.ensure(a, 8, 1)
    core.release_pages(b)
    assert core.pages_free() == 2 and core.table(b) == [] and core.ensure(a, 8, 1)


def test_misuse_is_refused():
    core = HostCore([(4, 4, 0)], max_requests=1)
    a = core.acquire_slot()
    with pytest.raises(CoreError, match="no free request slot"):
        core.acquire_slot()
    core.release_slot(a)
    with pytest.raises(CoreError, match="not in use"):
        core.release_slot(a)
    with pytest.raises(CoreError, match="not in use"):
        core.ensure(a, 0, 1)
    with pytest.raises(CoreError):
        HostCore([(0, 4, 0)], max_requests=1)


def test_window_group_gives_pages_back():
    # group 0 keeps every key, group 1 only the last 6; pages of 4
    core = HostCore([(4, 64, 0), (4, 64, 6)], max_requests=2)
    s = core.acquire_slot()
    pos = 0
    for n in (5, 1, 1, 7, 1, 1, 1, 9, 1):
        assert core.ensure(s, pos, n)
        t0, t1 = core.table(s, 0), core.table(s, 1)
        assert len(t0) == len(t1) == -(-(pos + n) // 4) and all(p >= 0 for p in t0)
        first_visible = max(0, pos + 1 - 6)          # oldest key the query at `pos` sees
        for i, page in enumerate(t1):
            assert (page >= 0) == (i >= first_visible // 4), f"pos {pos}: logical page {i} -> {page}"
        pos += n
        check_invariants(core, [s])
    assert core.pages_held(s, 1) < core.pages_held(s, 0)
    core.release_slot(s)
    assert core.pages_free(0) == 64 and core.pages_free(1) == 64


def test_window_pages_are_used_again_by_the_same_request():
    core = HostCore([(4, 3, 5)], max_requests=1)     # 3 pages only: a long request lives on reuse
    s = core.acquire_slot()
    seen = []
    for pos in range(40):
        assert core.ensure(s, pos, 1), f"position {pos}"
        seen.append(core.table(s)[-1])
    assert set(seen) == {0, 1} and core.pages_held(s) <= 2, "five keys never span more than two pages of four"


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests(seed):
    rng = random.Random(seed)
    groups = [(4, 40, 0), (4, 30, 9)] if seed % 2 else [(16, 12, 0)]
    core = HostCore(groups, max_requests=6)
    live = {}
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 6:
            live[core.acquire_slot()] = 0
        elif action < 0.85 and live:
            s = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 17])
            before = [core.pages_free(g) for g in range(core.n_groups)]
            tables = [core.table(s, g) for g in range(core.n_groups)]
            if core.ensure(s, live[s], n):
                live[s] += n
            else:
                held = [[p for p in t if p >= 0] for t in tables]
                now = [[p for p in core.table(s, g) if p >= 0] for g in range(core.n_groups)]
                assert all(set(n_) <= set(h) for n_, h in zip(now, held)), "a failed ensure took a page"
        elif action < 0.93 and live:
            s = rng.choice(list(live))
            core.release_pages(s)
            live[s] = 0
        elif live:
            s = rng.choice(list(live))
            core.release_slot(s)
            del live[s]
        check_invariants(core, list(live))
    for s in list(live):
        core.release_slot(s)
    assert all(core.pages_free(g) == core.pages_total(g) for g in range(core.n_groups)) and core.slots_in_use() == 0


def test_batch_words():
    """The flattened batch (src/batch.rs:20-49, src/serve/engine.rs:96-154): positions,
    q_starts, seq_lens, slot map through the block table, padded tables."""
    core = HostCore([(4, 16, 0)], max_requests=4)
    a, b = core.acquire_slot(), core.acquire_slot()
    assert core.ensure(b, 0, 6) and core.ensure(a, 0, 3) and core.ensure(b, 6, 1)
    words = np.zeros(256, dtype=np.int32)
    off = core.build_batch([a, b], [0, 6], [3, 1], [11, 12, 13, 21], [2, 3], words)
    T, R = 4, 2
    assert words[off.header:off.header + 3].tolist() == [T, R, 2]
    assert words[off.tokens:off.tokens + T].tolist() == [11, 12, 13, 21]
    assert words[off.positions:off.positions + T].tolist() == [0, 1, 2, 6]
    assert words[off.token_entry:off.token_entry + T].tolist() == [0, 0, 0, 1]
    assert words[off.q_starts:off.q_starts + R + 1].tolist() == [0, 3, 4]
    assert words[off.seq_lens:off.seq_lens + R].tolist() == [3, 7]
    assert words[off.slots:off.slots + R].tolist() == [a, b]
    assert words[off.want_rows:off.want_rows + 2].tolist() == [2, 3]
    ta, tb = core.table(a), core.table(b)
    assert tb == [0, 1] and ta == [2]
    w = off.widths[0]
    assert w == 2
    assert words[off.tables[0]:off.tables[0] + R * w].tolist() == [ta[0], 0, tb[0], tb[1]]
    assert words[off.slot_maps[0]:off.slot_maps[0] + T].tolist() == [ta[0] * 4, ta[0] * 4 + 1, ta[0] * 4 + 2, tb[1] * 4 + 2]
    with pytest.raises(CoreError, match="has no page"):
        core.build_batch([a], [3], [2], [1, 2], [], words)       # position 4 was never ensured
    with pytest.raises(CoreError, match="words"):
        core.build_batch([a], [0], [3], [1, 2, 3], [], np.zeros(4, dtype=np.int32))


def test_pool_sizes_from_memory_give_a_window_only_what_it_can_hold():
    """Two groups, one with a window: the windowed one is given what `max_requests` requests can hold at once (the
    window, a step's portion, and a page for where the span starts), the other the rest, and the most any request
    ever holds in the windowed group (measured on the host core, portion after portion) stays within its share."""
    import torch
    from llm_rs_amd.cache import CacheManager, PagedKV
    full, windowed = PagedKV(2, 32), PagedKV(2, 32, window=40)
    needs = [(full, None), (windowed, None), (full, None), (windowed, 1)]        # the last run reads run 1's cache
    page, requests, seq, step = 16, 4, 4096, 48
    per_page = lambda layers: layers * 2 * (32 + 32) * 2 * page
    budget = 3_000_000
    got = CacheManager.pages_that_fit(needs, torch.bfloat16, page, 2 * budget, 0.5, requests, seq, step)
    assert got[1] == requests * -(-(40 + step + page) // page) == 28
    assert got[0] == (budget - got[1] * per_page(1)) // per_page(2)
    assert got[0] * per_page(2) + got[1] * per_page(1) <= budget < (got[0] + 1) * per_page(2) + got[1] * per_page(1)
    # with memory to spare nobody gets more than the requests can fill; with next to none, one page each
    assert CacheManager.pages_that_fit(needs, torch.bfloat16, page, 1 << 40, 0.9, requests, seq, step) == [requests * seq // page, 28]
    assert CacheManager.pages_that_fit(needs, torch.bfloat16, page, 1000, 0.9, requests, seq, step) == [1, 1]
    # without the step's size a portion may be a whole sequence: no less than the other group then
    assert CacheManager.pages_that_fit(needs, torch.bfloat16, page, 1 << 40, 0.9, requests, seq) == [requests * seq // page] * 2
    core = HostCore([(page, got[0], 0), (page, got[1], 40)], requests, step * requests, step, seq)
    slots = [core.acquire_slot() for _ in range(requests)]
    rng = random.Random(3)
    at = [0] * requests
    for _ in range(200):
        for s in slots:
            n = rng.randint(1, step)
            assert core.ensure(s, at[s], n), "the windowed group ran out although sized for the worst case"
            at[s] += n
            assert core.pages_held(s, 1) <= got[1] // requests
        if max(at) + step > got[0] // requests * page:
            break
    check_invariants(core, slots)
