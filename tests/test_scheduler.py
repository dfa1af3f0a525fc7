"""The scheduler's decisions, on the host alone: a stand-in model makes each
next token a function of the request's whole token sequence so far, so outputs
can be checked against a one-request-at-a-time run whatever the batching.
Reference: src/serve/scheduler.rs:34-76 and the loop of src/serve/engine.rs:161-231."""
import numpy as np
import pytest

from llm_rs_amd.cache import CoreError, HostCore


def next_token(tokens):
    h = 1469598103934665603
    for t in tokens:
        h = ((h ^ (t + 1)) * 1099511628211) % (1 << 64)
    return int(h % 97)


class Driver:
    """Runs the plan/build/commit loop with the stand-in model."""

    def __init__(self, core):
        self.core, self.words = core, np.zeros(1 << 16, dtype=np.int32)
        self.seen = {}          # slot -> tokens fed so far (what the cache would hold)
        self.steps = []

    def step(self):
        core = self.core
        plan = core.plan()
        if not plan:
            return []
        off, T, n_want = core.build_planned(self.words)
        toks = self.words[off.tokens:off.tokens + T].tolist()
        pos = self.words[off.positions:off.positions + T].tolist()
        sampled, at = [], 0
        for slot, start, count, samples in plan:
            if start == 0:
                self.seen[slot] = []
            assert pos[at:at + count] == list(range(start, start + count))
            assert len(self.seen[slot]) == start, "a portion must start where the cache ends"
            self.seen[slot] += toks[at:at + count]
            at += count
            if samples:
                sampled.append(next_token(self.seen[slot]))
        want = self.words[off.want_rows:off.want_rows + n_want].tolist()
        ends = np.cumsum([p[2] for p in plan]) - 1
        assert want == [int(e) for e, p in zip(ends, plan) if p[3]]
        self.steps.append(plan)
        return core.commit(sampled)

    def run(self, limit=10000):
        done = {}
        for _ in range(limit):
            if self.core.idle():
                return done
            for slot in self.step():
                done[slot] = (self.core.request_output(slot), self.core.request_info(slot))
                self.core.drop_request(slot)
        raise AssertionError("the scheduler did not finish")


def alone(prompt, max_new, stop=()):
    tokens, out = list(prompt), []
    for _ in range(max_new):
        t = next_token(tokens)
        if t in stop:
            return out, "stop"
        out.append(t); tokens.append(t)
    return out, "length"


def test_budget_portions_and_order():
    core = HostCore([(4, 1000, 0)], max_requests=8, token_budget=16, max_chunk=0)
    a = core.add_request(list(range(20)), 3)
    b = core.add_request(list(range(5)), 3)
    c = core.add_request(list(range(7)), 3)
    d = Driver(core)
    d.step()
    assert d.steps[-1] == [(a, 0, 16, False)], "the budget cuts the first prompt"
    d.step()
    assert d.steps[-1] == [(a, 16, 4, True), (b, 0, 5, True), (c, 0, 7, True)], "running first, then waiting in arrival order"
    d.step()
    assert d.steps[-1] == [(a, 20, 1, True), (b, 5, 1, True), (c, 7, 1, True)], "decoding: one token each"
    for plan in d.steps:
        assert sum(p[2] for p in plan) <= 16


def test_max_chunk_caps_one_request():
    core = HostCore([(4, 1000, 0)], max_requests=8, token_budget=64, max_chunk=8)
    a = core.add_request(list(range(20)), 2)
    b = core.add_request(list(range(3)), 2)
    d = Driver(core)
    d.step(); d.step(); d.step()
    assert d.steps[0] == [(a, 0, 8, False), (b, 0, 3, True)]
    assert d.steps[1] == [(a, 8, 8, False), (b, 3, 1, True)]
    assert d.steps[2][0] == (a, 16, 4, True)


def test_outputs_do_not_depend_on_batching_and_finish_reasons():
    core = HostCore([(4, 1000, 0)], max_requests=4, token_budget=24, max_chunk=10)
    prompts = [[3, 1, 4, 1, 5], list(range(30)), [9], [2, 7, 1, 8, 2, 8], [6] * 13]
    stop = [5, 11]
    d, slots, pending = Driver(core), {}, list(enumerate(prompts))
    done = {}
    while pending or not core.idle():
        while pending:
            s = core.add_request(pending[0][1], 12, stop=stop)
            if s < 0:
                break
            slots[s] = pending.pop(0)[0]
        for s in d.step():
            done[slots.pop(s)] = (core.request_output(s), core.request_info(s)["finish"])
            core.drop_request(s)
    for i, p in enumerate(prompts):
        out, reason = alone(p, 12, stop)
        assert done[i][0] == out and done[i][1] == (1 if reason == "stop" else 2)
        assert len(out) <= 12
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0


def test_exactly_max_new_tokens_without_an_extra_step():
    core = HostCore([(4, 100, 0)], max_requests=2, token_budget=64)
    core.add_request([1, 2, 3], 4)
    d = Driver(core)
    done = d.run()
    (out, info), = done.values()
    assert len(out) == 4 and info["finish"] == 2
    assert len(d.steps) == 4, "prompt step samples the first token; three decode steps give the rest"


def test_pages_run_out_skip_and_head_of_line():
    # 6 pages of 4.  a takes 3, b takes 3; c must wait at the head of the line, and d behind it,
    # although d alone would fit later.
    core = HostCore([(4, 6, 0)], max_requests=8, token_budget=64)
    a = core.add_request(list(range(10)), 2)      # 11 positions -> 3 pages
    b = core.add_request(list(range(9)), 3)       # 11 positions -> 3 pages
    c = core.add_request(list(range(6)), 2)
    e = core.add_request([1], 1)
    d = Driver(core)
    d.step()
    assert [p[0] for p in d.steps[-1]] == [a, b] and core.num_waiting() == 2, "c does not fit; e stays behind c"
    d.step()                                          # a finishes (2 tokens), its pages come back
    d.step()
    assert c in [p[0] for p in d.steps[-1]], "c is admitted once pages are free"
    done = d.run()
    assert core.pages_free() == 6 and core.preemptions() == 0


def test_preemption_when_nobody_can_advance():
    # Two requests fit at admission but not at their full length: when both need a new
    # page and none is free, the one admitted last gives its pages back, waits, and is
    # computed again from its prompt and what it generated; its output does not change.
    core = HostCore([(4, 5, 0)], max_requests=4, token_budget=64)
    pa, pb = list(range(8)), list(range(20, 27))
    a = core.add_request(pa, 9)       # 16 positions -> 4 pages at the end
    b = core.add_request(pb, 9)
    d = Driver(core)
    done = d.run()
    assert core.preemptions() >= 1
    assert done[a][0] == alone(pa, 9)[0] and done[b][0] == alone(pb, 9)[0]
    assert done[b][1]["preemptions"] >= 1 and done[a][1]["preemptions"] == 0, "the request admitted last is the one that yields"
    restarts = [p for plan in d.steps for p in plan if p[0] == b and p[1] == 0]
    assert len(restarts) >= 2 and restarts[-1][2] > len(pb), "the recomputed portion holds prompt and generated tokens"
    assert core.pages_free() == 5


def test_a_request_that_can_never_fit_is_an_error_not_a_spin():
    core = HostCore([(4, 5, 0)], max_requests=4, token_budget=64, max_positions=64)
    with pytest.raises(CoreError, match="pages"):
        core.add_request(list(range(18)), 4)          # 21 positions -> 6 pages > 5
    with pytest.raises(CoreError, match="positions"):
        core.add_request(list(range(60)), 10)
    with pytest.raises(CoreError, match="prompt"):
        core.add_request([], 4)
    assert core.idle() and core.slots_in_use() == 0


def test_request_table_full_means_ask_again():
    core = HostCore([(4, 100, 0)], max_requests=2, token_budget=64)
    assert core.add_request([1], 2) >= 0 and core.add_request([2], 2) >= 0
    assert core.add_request([3], 2) == -1
    Driver(core).run()
    assert core.add_request([3], 2) >= 0


@pytest.mark.parametrize("seed", range(5))
def test_random_load_with_a_small_pool(seed):
    rng = np.random.default_rng(seed)
    core = HostCore([(4, 14, 0)], max_requests=5, token_budget=int(rng.integers(8, 40)), max_chunk=int(rng.integers(0, 9)))
    prompts = [rng.integers(0, 50, int(rng.integers(1, 25))).tolist() for _ in range(12)]
    news = [int(rng.integers(1, 12)) for _ in prompts]
    d, slots, pending, done = Driver(core), {}, list(range(12)), {}
    for _ in range(5000):
        while pending:
            s = core.add_request(prompts[pending[0]], news[pending[0]])
            if s < 0:
                break
            slots[s] = pending.pop(0)
        if core.idle() and not pending:
            break
        for s in d.step():
            done[slots.pop(s)] = core.request_output(s)
            core.drop_request(s)
        held = sum(core.pages_held(s) for s in slots)
        assert held + core.pages_free() == 14
    assert sorted(done) == list(range(12))
    for i in range(12):
        assert done[i] == alone(prompts[i], news[i])[0], f"request {i}"
    assert core.pages_free() == 14


def test_sampling_words_and_generator():
    """The uniform a request draws comes from its own xorshift64 stream
    (src/sampler/mod.rs:2-25): seed 42 by default, seed 0 -> 0xDEADBEEFCAFE."""
    from llm_rs_amd.cache import xorshift64_stream
    from plain_llama import PlainXorshift
    for seed in (42, 0, 7, 2**63 + 5):
        g = PlainXorshift(seed)
        assert xorshift64_stream(seed, 5) == [g.next_u64() for _ in range(5)]
    x = 42
    x ^= (x << 13) & (2**64 - 1); x ^= x >> 7; x ^= (x << 17) & (2**64 - 1)
    assert xorshift64_stream(42, 1) == [x]
    core = HostCore([(4, 100, 0)], max_requests=2, token_budget=64)
    core.add_request([1, 2], 3, temperature=0.8, top_k=40, top_p=0.9, seed=42)
    words = np.zeros(4096, dtype=np.int32)
    g = PlainXorshift(42)
    for step in range(3):
        core.plan()
        off, T, n_want = core.build_planned(words)
        w = words[off.sampling:off.sampling + 4]
        assert w[0:1].view(np.float32)[0] == np.float32(g.next_f32())
        assert w[1:2].view(np.float32)[0] == np.float32(0.8) and w[2] == 40 and w[3:4].view(np.float32)[0] == np.float32(0.9)
        core.commit([5])


def test_abort_gives_everything_back():
    core = HostCore([(4, 20, 0)], max_requests=3, token_budget=8)
    a = core.add_request(list(range(10)), 5)
    b = core.add_request(list(range(6)), 5)
    d = Driver(core)
    d.step()                      # a runs its first portion, b still waits
    core.abort_request(a)
    core.abort_request(b)
    assert core.idle() and core.pages_free() == 20 and core.slots_in_use() == 0
    with pytest.raises(CoreError, match="holds no request"):
        core.abort_request(a)
    c = core.add_request([1, 2, 3], 2)
    assert Driver(core).run()[c][0] == alone([1, 2, 3], 2)[0]


def test_window_group_bound_holds_for_portions_that_start_anywhere():
    """With a window, a request's pages at once are the keys its portion's first query still sees and
    the portion itself.  Where a portion starts depends on what else shared the budget: page 16,
    window 16, portions of 16 need 2 pages from an aligned start and 3 from position 17.  A request
    is admitted only to a pool that holds the worst start."""
    with pytest.raises(CoreError, match="3 pages"):
        HostCore([(16, 2, 16)], max_requests=2, token_budget=16, max_chunk=16).add_request(list(range(40)), 8)
    # a request shorter than window + portion needs no more than all its keys
    small = HostCore([(16, 2, 16)], max_requests=2, token_budget=16, max_chunk=16)
    small.check_request(20, 13)                 # 32 computed positions: 2 pages
    # two requests share the budget, so portions start off the page grid; the pool is exactly the bound
    core = HostCore([(16, 3, 16)], max_requests=2, token_budget=17, max_chunk=16)
    a = core.add_request([1] * 3, 2)            # one token of the budget goes to this one while it decodes
    b = core.add_request(list(range(60)), 6)
    d = Driver(core)
    done = d.run()
    starts = [p[1] for plan in d.steps for p in plan if p[0] == b]
    assert any(s % 16 for s in starts), "the case must cut portions off the page grid"
    assert done[a][0] == alone([1] * 3, 2)[0] and done[b][0] == alone(list(range(60)), 6)[0]
    assert done[b][1]["preemptions"] == 0
    assert core.pages_free() == 3


def test_check_request_changes_nothing():
    core = HostCore([(4, 5, 0)], max_requests=4, token_budget=64, max_positions=64)
    with pytest.raises(CoreError, match="pages"):
        core.check_request(18, 4)
    core.check_request(10, 4)
    assert core.idle() and core.slots_in_use() == 0 and core.pages_free() == 5


class AheadDriver:
    """The loop of a caller that keeps one step in flight: a step is started (its samples are not known to the
    scheduler yet), the next one is planned and started, then the first one's samples are committed.  The stand-in
    device puts a sample of the step in flight where the plan ahead names it."""

    def __init__(self, core):
        self.core, self.words = core, np.zeros(1 << 16, dtype=np.int32)
        self.seen = {}            # slot -> tokens fed so far
        self.flight = None        # samples of the step in flight
        self.wasted = 0           # tokens run for a request that had ended

    def start(self):
        """Plans and 'runs' a step; returns its samples, or None when nothing could be planned."""
        core = self.core
        plan = core.plan()
        if not plan:
            return None
        sources = core.plan_sources()
        off, T, n_want = core.build_planned(self.words)
        toks = self.words[off.tokens:off.tokens + T].tolist()
        sampled, at = [], 0
        for (slot, start, count, samples), src in zip(plan, sources):
            if src >= 0:
                assert count == 1 and samples and self.flight is not None
                toks[at] = self.flight[src]                 # what the device does
            if start == 0:
                self.seen[slot] = []
            assert len(self.seen[slot]) == start, "a portion must start where the cache ends"
            self.seen[slot] = self.seen[slot] + toks[at:at + count]
            at += count
            if samples:
                sampled.append(next_token(self.seen[slot]))
        return sampled

    def step(self):
        """One turn of the loop; returns the slots that finished."""
        core = self.core
        if self.flight is None:
            self.flight = self.start()
            if self.flight is None:
                return []
            core.launch()
        ahead = self.start()                                   # before the step in flight is committed
        finished = core.commit(self.flight)
        self.flight = ahead
        if ahead is not None:
            core.launch()
        return finished


@pytest.mark.parametrize("seed", range(8))
def test_one_step_ahead_gives_the_same_outputs(seed):
    """Random load, small pool, stop tokens: with a step in flight while the next is planned every request's output
    and finish reason are what it gets alone; no page is lost; a request that ends on a stop token costs one token
    run for nothing and no more."""
    rng = np.random.default_rng(100 + seed)
    pages = 16
    core = HostCore([(4, pages, 0)], max_requests=5, token_budget=int(rng.integers(8, 40)), max_chunk=int(rng.integers(0, 9)))
    n = 14
    prompts = [rng.integers(0, 50, int(rng.integers(1, 25))).tolist() for _ in range(n)]
    news = [int(rng.integers(1, 14)) for _ in prompts]
    stops = [rng.integers(0, 97, int(rng.integers(0, 12))).tolist() for _ in prompts]
    d, slots, pending, done = AheadDriver(core), {}, list(range(n)), {}
    for _ in range(5000):
        while pending:
            s = core.add_request(prompts[pending[0]], news[pending[0]], stop=stops[pending[0]])
            if s < 0:
                break
            slots[s] = pending.pop(0)
        if core.idle() and not pending and d.flight is None:
            break
        for s in d.step():
            info = core.request_info(s)
            done[slots.pop(s)] = (core.request_output(s), "stop" if info["finish"] == 1 else "length")
            core.drop_request(s)
        held = sum(core.pages_held(s) for s in slots)
        assert held + core.pages_free() == pages
    assert sorted(done) == list(range(n))
    for i in range(n):
        assert done[i] == alone(prompts[i], news[i], stops[i]), f"request {i}"
    assert core.pages_free() == pages and not core.in_flight()


def test_one_step_ahead_plans_the_token_in_flight_and_drops_what_a_stop_wasted():
    core = HostCore([(4, 20, 0)], max_requests=3, token_budget=16)
    first = next_token([1, 2, 3])
    a = core.add_request([1, 2, 3], 5, stop=[next_token([1, 2, 3, first])])      # ends on its second sample
    b = core.add_request([4, 5], 1)                                              # its first sample is its last
    assert core.plan() == [(a, 0, 3, True), (b, 0, 2, True)]
    assert core.plan_sources() == [-1, -1]
    words = np.zeros(4096, dtype=np.int32)
    core.build_planned(words)
    core.launch()
    assert core.in_flight()
    # ahead: a's next token is row 0 of the step in flight; b is not planned, the token in flight is its last
    assert core.plan() == [(a, 3, 1, True)] and core.plan_sources() == [0]
    off, T, n_want = core.build_planned(words)
    assert (T, n_want) == (1, 1)
    assert core.commit([first, 9]) == [b]
    assert core.request_output(b) == [9]
    core.drop_request(b)
    core.launch()
    # the step after: a's second sample is in flight
    assert core.plan() == [(a, 4, 1, True)] and core.plan_sources() == [0]
    core.build_planned(words)
    assert core.commit([next_token([1, 2, 3, first])]) == [a]                    # the stop token: a ends here
    assert core.request_output(a) == [first] and core.request_info(a)["finish"] == 1
    core.drop_request(a)
    core.launch()                                                                # what was planned for it is dead
    assert core.plan() == []
    assert core.commit([55]) == []                                               # its sample is dropped
    assert core.idle() and core.pages_free() == 20 and core.slots_in_use() == 0 and not core.in_flight()


def test_nobody_is_preempted_ahead_of_a_step_in_flight():
    core = HostCore([(4, 2, 0)], max_requests=2, token_budget=16)
    a = core.add_request([1, 2, 3, 4], 5)
    b = core.add_request([5, 6, 7, 8], 5)
    words = np.zeros(4096, dtype=np.int32)
    assert core.plan() == [(a, 0, 4, True), (b, 0, 4, True)]
    core.build_planned(words)
    core.launch()
    assert core.plan() == [] and core.preemptions() == 0      # both need a second page and none is free: the caller lands the step first
    assert core.commit([11, 12]) == []
    plan = core.plan()                                        # in turn again: the request admitted last gives way
    assert plan == [(a, 4, 1, True)] and core.preemptions() == 1


@pytest.mark.parametrize("seed", range(6))
def test_one_step_ahead_with_requests_aborted_at_any_time(seed):
    """Requests are aborted between the turns of the loop, also while the step in flight holds an entry of theirs and
    after the step ahead was planned with one: what they sampled is dropped, their slot may go to the next request
    at once, no page is lost, and every request that was not aborted gets the output it gets alone."""
    rng = np.random.default_rng(500 + seed)
    pages = 18
    core = HostCore([(4, pages, 0)], max_requests=4, token_budget=int(rng.integers(6, 30)), max_chunk=int(rng.integers(0, 7)))
    n = 16
    prompts = [rng.integers(0, 50, int(rng.integers(1, 20))).tolist() for _ in range(n)]
    news = [int(rng.integers(1, 12)) for _ in prompts]
    stops = [rng.integers(0, 97, int(rng.integers(0, 6))).tolist() for _ in prompts]
    doomed = {int(i): int(rng.integers(0, 8)) for i in rng.choice(n, 5, replace=False)}     # request -> turns it lives
    d, slots, pending, done, age, aborted = AheadDriver(core), {}, list(range(n)), {}, {}, set()
    for _ in range(5000):
        while pending:
            s = core.add_request(prompts[pending[0]], news[pending[0]], stop=stops[pending[0]])
            if s < 0:
                break
            slots[s] = pending.pop(0)
            age[slots[s]] = 0
        if core.idle() and not pending and d.flight is None:
            break
        for s in d.step():
            info = core.request_info(s)
            done[slots.pop(s)] = (core.request_output(s), "stop" if info["finish"] == 1 else "length")
            core.drop_request(s)
        for s, r in list(slots.items()):
            age[r] += 1
            if r in doomed and age[r] > doomed[r]:
                core.abort_request(s)
                aborted.add(slots.pop(s))
        held = sum(core.pages_held(s) for s in slots)
        assert held + core.pages_free() == pages
    assert sorted(list(done) + list(aborted)) == list(range(n)) and aborted
    for i in done:
        assert done[i] == alone(prompts[i], news[i], stops[i]), f"request {i}"
    assert core.pages_free() == pages and core.slots_in_use() == 0 and not core.in_flight()
