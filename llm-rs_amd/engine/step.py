"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.  Prompt portions and single decoded tokens are the same
thing here, entries of `count` tokens from position `start`, and all run as one
batch from the cache that earlier steps left (src/model.rs:5-8 `forward`, with
the batch of src/batch.rs:5-16 built as in src/serve/engine.rs:96-154).

Host work per step: ask the core for pages, let it flatten the batch into one
block of words in pinned memory, copy that block to the device once, launch.
Activations live in a workspace that grows to the largest step seen and is then
reused, so steady-state steps allocate nothing.

Steps in which every entry brings one token (decoding) are launch-bound: a few
hundred small kernels.  Such a step is recorded once into a HIP graph, keyed by
its batch size and block-table width, and replayed afterwards: the flattened
batch has the same layout for the same key, every kernel reads positions, tables
and counts from that block on the device, and nothing in the graph depends on
host values.  Grids that depend on the context length are recorded for the
width's capacity and leave early.
"""
from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import gc
import os
import weakref

import numpy as np
import torch

from ..cache import CacheManager


class OutOfPages(RuntimeError):
    pass


class _GrewWhileRecording(Exception):
    """A buffer would have had to grow in the middle of a recording."""


@dataclass
class StepEntry:
    slot: int
    start: int
    tokens: Sequence[int]
    want: Sequence[int] = ()      # places among `tokens` whose logits are wanted


class StepContext:
    """What parts see of the running step.  Device arrays are int32."""

    def __init__(self, runner: "StepRunner"):
        # (not a reference that counts: runner and context would hold each other, and a dropped engine,
        # with its recorded graphs and device memory, would wait for the cycle collector)
        self._runner = weakref.proxy(runner)
        self.n_tokens = 0
        self.n_entries = 0
        self.n_want = 0
        self.run_index = -1
        self.tokens = self.positions = self.token_entry = None
        self.q_starts = self.seq_lens = self.slots = self.want_rows = self.sampling = None
        self.slot_maps: List[torch.Tensor] = []
        self.block_tables: List[torch.Tensor] = []
        self.entries: List[Tuple[int, int, int]] = []   # host copy: (slot, start, count)
        self.max_seq_len = 0                            # largest start + count among the entries
        self.n_single = 0                               # entries that bring one token
        self.single_lens: List[int] = []                # their lengths with that token
        self._keys_seen = {}
        self.serial = 0                                 # counts the steps bound to this context
        self.part_state = {}                            # what parts keep from step to step, by `recording_signature`
        self.device = runner.device
        # A norm without a kernel of its own (steps of a few tokens): the part that adds into the stream last
        # before a norm leaves what that norm needs (`room_for_next_norm`, `note_left`), and the norm hands it on
        # to the product that follows (`left_for`).  `upcoming_norm` is the norm that will read the stream after
        # the part that runs now (its block says so); `norm_after_block` the one after the block (the model says so).
        self.upcoming_norm = None
        self.norm_after_block = None
        self.wants_every_row = False
        self._left = None               # kernels.NextNorm that describes the stream as it stands, or None
        self._left_of = 0               # the stream it describes
        self._last_y = 0                # where the rows left last lie

    def workspace(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        return self._runner.workspace(name, shape, dtype)

    def single_keys(self, window: int = 0) -> int:
        """How many keys the single-token entries see together, each through a window of `window` keys (0: all)."""
        got = self._keys_seen.get(window)
        if got is None:
            got = sum(self.single_lens) if window <= 0 else sum(min(n, window) for n in self.single_lens)
            self._keys_seen[window] = got
        return got

    def room_for_next_norm(self, h: torch.Tensor, w: torch.Tensor):
        """For a part about to add a product with weight `w` into the stream `h`: a `kernels.NextNorm` for that
        product to fill (`kernels().gemm(..., leave=...)`; then `note_left(h, it)`), or None when the norm that
        follows cannot be left to the next product (no such norm, other dtype, too many rows)."""
        from ..kernels import NextNorm, kernels
        norm = self.upcoming_norm
        weight = norm.deferred_weight() if norm is not None else None
        T, N = h.shape[0], w.shape[0]
        if weight is None or N != h.shape[1] or weight.shape[0] != N:
            return None
        plan = kernels().norm_left_by_product(T, N, w.shape[1], w.dtype)
        if plan is None:
            return None
        if not plan.whole:
            return NextNorm(self._prenormed(T, N), self.workspace("model.sumsq", (T, plan.parts), torch.float32), weight)
        eps = norm.deferred_eps()
        return NextNorm(self._prenormed(T, N), None, weight, eps) if eps is not None and eps > 0 else None

    def _prenormed(self, T: int, N: int) -> torch.Tensor:
        """Room for the rows a product leaves: not the rows that were left last, which the part at work may
        still be reading as its input."""
        y = self.workspace("model.prenormed", (T, N), torch.bfloat16)
        if self._last_y == y.data_ptr():
            y = self.workspace("model.prenormed.other", (T, N), torch.bfloat16)
        return y

    def note_left(self, h: torch.Tensor, left) -> None:
        """`left` (a filled NextNorm, or None) is what describes `h` from now on."""
        self._left, self._left_of = left, (h.data_ptr() if left is not None else 0)
        if left is not None:
            self._last_y = left.y.data_ptr()

    def left_for(self, h: torch.Tensor):
        """What the last product that added into `h` left for the norm that follows, or None."""
        return self._left if self._left is not None and self._left_of == h.data_ptr() else None

    def gemm_workspace(self, a: torch.Tensor, w: torch.Tensor) -> Optional[torch.Tensor]:
        """Room for the partial sums of a @ w.T, when the kernel would split K over blocks."""
        from ..kernels import kernels
        n = kernels().gemm_workspace_floats(a.shape[0], w.shape[0], w.shape[1])
        return self.workspace("gemm.partial", (n,), torch.float32) if n else None


class StepRunner:
    def __init__(self, model, cache: CacheManager, device, words_capacity: int = 1 << 16):
        self.model, self.cache, self.device = model, cache, torch.device(device)
        self._buffers: Dict[str, torch.Tensor] = {}
        self._pinned = self.device.type == "cuda"
        self._host = [self._new_host(words_capacity) for _ in range(2)]
        self._events = [None, None]
        self._turn = 0
        self._dev_words = torch.zeros(words_capacity, dtype=torch.int32, device=self.device)
        self.ctx = StepContext(self)
        # HIP graphs of decode steps: key -> (graph, logits); a key is recorded when it has been seen a few times
        # (fixed-size state does not stand in the way: it is reset before a step runs, outside any recording,
        # and a mixer that says it is graph_safe finds its rows through the slots on the device)
        self.use_graphs = (self._pinned and os.environ.get("LLMRS_GRAPHS", "1") != "0" and not os.environ.get("LLM_PERF")
                           and bool(getattr(model, "graph_safe", lambda: False)()))
        # With this on, an event is recorded right before a step's first kernel, for whoever wants the
        # device's share of the time (the engine pairs it with one after sampling).
        self.time_device = False
        self.started: Optional["torch.cuda.Event"] = None
        self.max_graph_batch = 512
        self.max_graphs = 256            # recorded graphs kept (the least recently replayed goes first)
        self._graphs: "OrderedDict[tuple, tuple]" = OrderedDict()
        self._seen: Dict[tuple, int] = {}
        self._recording = False          # between the start and the end of a stream capture
        self.graph_replays = 0

    def _new_host(self, n: int) -> torch.Tensor:
        return torch.zeros(n, dtype=torch.int32, pin_memory=self._pinned)

    def workspace(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * dtype.itemsize
        buf = self._buffers.get(name)
        if buf is None or buf.numel() < nbytes:
            if self._recording:
                # Neither allocating nor dropping the recorded graphs (they hold the old addresses) may
                # happen while a stream is being captured: give the recording up; the step then runs
                # eagerly, where this buffer grows in the ordinary way.
                raise _GrewWhileRecording(name)
            # grow with head room so that a slowly growing step does not reallocate each time
            cap = max(nbytes, 256) if buf is None else max(nbytes, 2 * buf.numel())
            buf = torch.empty(cap, dtype=torch.uint8, device=self.device)
            self._buffers[name] = buf
            self._drop_graphs()         # recorded graphs hold the old addresses
        return buf[:nbytes].view(dtype).view(*shape)

    def _drop_graphs(self) -> None:
        """Forgets every recorded graph.  Destroying a graph frees device objects, so never during a recording."""
        assert not self._recording, "recorded graphs must not be destroyed while a stream is being captured"
        self._settle()
        self._graphs.clear()
        self._seen.clear()

    def _settle(self) -> None:
        """Waits for what has been started on the device, before a recorded graph is destroyed: with a step in flight
        while the next is planned, the graph being destroyed may be the one that is running.  (Rare: buffers grow a
        few times in an engine's life, and recordings are dropped when a new one takes the oldest one's place.)"""
        if self._graphs and self._pinned:
            torch.cuda.current_stream(self.device).synchronize()

    # -- staging -----------------------------------------------------------------
    def _staging(self, words_needed: int) -> np.ndarray:
        self._turn ^= 1
        i = self._turn
        if self._events[i] is not None:
            self._events[i].synchronize()
            self._events[i] = None
        if self._host[i].numel() < words_needed:
            self._host[i] = self._new_host(max(words_needed, 2 * self._host[i].numel()))
        return self._host[i].numpy()

    def _upload(self, n_words: int) -> torch.Tensor:
        i = self._turn
        if self._dev_words.numel() < n_words:
            self._dev_words = torch.zeros(max(n_words, 2 * self._dev_words.numel()), dtype=torch.int32, device=self.device)
            self._drop_graphs()
        dev = self._dev_words[:n_words]
        dev.copy_(self._host[i][:n_words], non_blocking=True)
        if self._pinned:
            ev = torch.cuda.Event()
            ev.record()
            self._events[i] = ev
        return dev

    def _estimate_words(self, T: int, R: int, n_want: int, longest: int, widths=None) -> int:
        """Upper bound of the flattened batch's size; `longest` is the largest start + count.
        A block table never has more entries than the positions ensured for it need."""
        words = 4 + 3 * T + 3 * R + 1 + 5 * n_want
        for g, grp in enumerate(self.cache.groups):
            words += T + R * (widths[g] if widths else max(1, -(-longest // grp.page_size)))
        return words + 16

    def _graph_widths(self, counts, longest: int):
        """Block-table widths to record a decode step with, or None when the step is not one
        that is recorded: every entry brings one token, and the batch is not huge."""
        if not self.use_graphs or len(counts) > self.max_graph_batch or any(c != 1 for c in counts):
            return None
        widths = []
        for grp in self.cache.groups:
            need = max(1, -(-longest // grp.page_size))
            cap = 64
            while cap < need:
                cap *= 2
            widths.append(cap)
        return widths

    def _bind(self, dev: torch.Tensor, off, T: int, R: int, n_want: int, entries, wants_all: bool = False) -> StepContext:
        c = self.ctx
        c.n_tokens, c.n_entries, c.n_want = T, R, n_want
        c.entries = entries
        c.wants_every_row = bool(wants_all)       # the wanted rows are the step's rows, each once and in order
        c.max_seq_len = max(start + count for _, start, count in entries)
        c.single_lens = [start + 1 for _, start, count in entries if count == 1]
        c.n_single = len(c.single_lens)
        c._keys_seen = {}
        c.serial += 1
        c.tokens = dev[off.tokens:off.tokens + T]
        c.positions = dev[off.positions:off.positions + T]
        c.token_entry = dev[off.token_entry:off.token_entry + T]
        c.q_starts = dev[off.q_starts:off.q_starts + R + 1]
        c.seq_lens = dev[off.seq_lens:off.seq_lens + R]
        c.slots = dev[off.slots:off.slots + R]
        c.want_rows = dev[off.want_rows:off.want_rows + n_want]
        c.sampling = dev[off.sampling:off.sampling + 4 * n_want].view(n_want, 4)
        c.slot_maps = [dev[o:o + T] for o in off.slot_maps]
        c.block_tables = [dev[o:o + R * w].view(R, w) for o, w in zip(off.tables, off.widths)]
        return c

    # -- the step ------------------------------------------------------------------
    def run(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Runs the entries' tokens as one batch; returns float32 logits
        [wanted, vocab] (a view into the workspace, valid until the next step), in
        the order of the entries and of their `want`, or None."""
        entries = [e for e in entries]
        if not entries:
            return None
        core = self.cache.core
        vocab = self.model.spec.vocab_size
        slots, starts, counts, tokens, want_rows = [], [], [], [], []
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"the entry of slot {e.slot} brings no tokens")
            if e.start + n > self.model.spec.max_positions:
                raise ValueError(f"slot {e.slot}: position {e.start + n - 1} is beyond the model's {self.model.spec.max_positions}")
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"slot {e.slot}: wanted place {w} is outside its {n} tokens")
                want_rows.append(len(tokens) + w)
            ids = np.asarray(e.tokens, dtype=np.int64)
            if ids.min() < 0 or ids.max() >= vocab:
                raise ValueError(f"slot {e.slot}: token ids must be in [0, {vocab}), got {int(ids.min())}..{int(ids.max())}")
            if not core.ensure(e.slot, e.start, n):
                raise OutOfPages(f"no cache pages left for slot {e.slot} at positions {e.start}..{e.start + n - 1}")
            slots.append(e.slot); starts.append(e.start); counts.append(n); tokens.extend(ids.tolist())
        T, R = len(tokens), len(entries)
        longest = max(a + b for a, b in zip(starts, counts))
        widths = self._graph_widths(counts, longest)
        words = self._staging(self._estimate_words(T, R, len(want_rows), longest, widths))
        off = core.build_batch(slots, starts, counts, tokens, want_rows, words, fixed_widths=widths)
        dev = self._upload(off.words)
        ctx = self._bind(dev, off, T, R, len(want_rows), list(zip(slots, starts, counts)), want_rows == list(range(T)))
        return self._execute(ctx, widths)

    def run_planned(self, samples_in_flight: Optional[torch.Tensor] = None):
        """Runs the step the scheduler planned; returns (logits or None, rows that sample, the plan).
        `samples_in_flight`: the ids (on the device) that the step before this one sampled, when the scheduler has
        not been told them yet: entries whose one token is among them get it there, on the device."""
        core = self.cache.core
        plan = core.plan()
        if not plan:
            return None, 0, plan
        T = sum(p[2] for p in plan)
        R = len(plan)
        longest = max(p[1] + p[2] for p in plan)
        rows, sources, at = [], [], 0
        if samples_in_flight is not None:
            for p, src in zip(plan, core.plan_sources()):
                if src >= 0:
                    rows.append(at); sources.append(src)
                at += p[2]
        widths = self._graph_widths([p[2] for p in plan], longest)
        words = self._staging(self._estimate_words(T, R, R, longest, widths) + 2 * len(rows))
        off, n_tokens, n_want = core.build_planned(words, fixed_widths=widths)
        n = len(rows)                              # behind the batch: where the samples in flight go, and which
        words[off.words:off.words + n] = rows
        words[off.words + n:off.words + 2 * n] = sources
        dev = self._upload(off.words + 2 * n)
        ctx = self._bind(dev, off, n_tokens, R, n_want, [(p[0], p[1], p[2]) for p in plan],
                         all(p[2] == 1 and p[3] for p in plan))
        if n:
            from ..kernels import kernels
            kernels().place_ids(ctx.tokens, dev[off.words:off.words + n], dev[off.words + n:off.words + 2 * n],
                                samples_in_flight, self.model.spec.vocab_size)
        return self._execute(ctx, widths), n_want, plan

    def _execute(self, ctx: StepContext, graph_widths=None) -> Optional[torch.Tensor]:
        fresh = [slot for slot, start, _ in ctx.entries if start == 0]
        self.cache.reset_state(fresh)
        if self.time_device and self._pinned:
            self.started = torch.cuda.Event(enable_timing=True)
            self.started.record()
        if graph_widths is None:
            return self.model.forward(ctx, self.cache.views)
        # A decode step.  Everything the kernels take from the host must be the same for
        # every step of this key: sizes, addresses, and the bound on the context length.
        ctx.max_seq_len = min(w * g.page_size for w, g in zip(graph_widths, self.cache.groups)) if graph_widths else ctx.max_seq_len
        key = (ctx.n_tokens, ctx.n_want, tuple(graph_widths), self._dev_words.data_ptr(), self.model.recording_key(ctx))
        hit = self._graphs.get(key)
        if hit is not None:
            self._graphs.move_to_end(key)
            hit[0].replay()
            self.graph_replays += 1
            return hit[1]
        # Recording costs about as much host time as ten eager steps save: a shape is recorded when it
        # keeps coming back (small batches, where the launches are what a step costs, sooner).
        self._seen[key] = self._seen.get(key, 0) + 1
        if self._seen[key] < (2 if ctx.n_tokens <= 64 else 4):
            return self.model.forward(ctx, self.cache.views)     # first times: run it, and let the workspace grow
        # Nothing may be destroyed on the device while a stream is being recorded: an object that the
        # cycle collector happened to free in the middle of it (another engine's graphs, say) ended the
        # process.  The collector rests meanwhile.
        graph = torch.cuda.CUDAGraph()
        was_enabled = gc.isenabled()
        gc.disable()
        gave_up = False
        self._recording = True
        try:
            with torch.cuda.graph(graph):
                logits = self.model.forward(ctx, self.cache.views)
        except _GrewWhileRecording:
            gave_up = True
        finally:
            self._recording = False
            if was_enabled:
                gc.enable()
        if gave_up:
            # A part asked for more room than the eager runs of this shape did.  The capture has ended;
            # what it recorded is dropped now, the step runs eagerly (its buffers grow there), and the
            # shape is counted from the start again.
            del graph
            self._seen.pop(key, None)
            return self.model.forward(ctx, self.cache.views)
        while len(self._graphs) >= self.max_graphs:
            self._settle()
            self._graphs.popitem(last=False)
        self._graphs[key] = (graph, logits)
        graph.replay()                  # recording does not run the kernels
        self.graph_replays += 1
        return logits
