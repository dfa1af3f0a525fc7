"""ctypes face of the host core (csrc/host): page pools, block tables, slots,
batch flattening and the scheduler, behind one handle."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_longlong, c_uint64, c_void_p
from typing import List, Sequence

import numpy as np

from ..csrc.build import load_host


class CoreError(RuntimeError):
    pass


_configured = False


def _lib():
    global _configured
    lib = load_host()
    if not _configured:
        lib.llmrs_core_create.restype = c_void_p
        lib.llmrs_core_create.argtypes = [c_int, POINTER(c_int), POINTER(c_int), POINTER(c_int), c_int, c_int, c_int, c_int]
        lib.llmrs_core_destroy.argtypes = [c_void_p]
        lib.llmrs_core_error.restype = c_char_p
        lib.llmrs_core_error.argtypes = [c_void_p]
        lib.llmrs_create_error.restype = c_char_p
        for name, args in {
            "llmrs_slot_acquire": [c_void_p], "llmrs_slot_release": [c_void_p, c_int],
            "llmrs_slots_in_use": [c_void_p],
            "llmrs_pages_free": [c_void_p, c_int], "llmrs_pages_total": [c_void_p, c_int],
            "llmrs_pages_held": [c_void_p, c_int, c_int],
            "llmrs_ensure": [c_void_p, c_int, c_int, c_int], "llmrs_release_pages": [c_void_p, c_int],
            "llmrs_table": [c_void_p, c_int, c_int, c_void_p, c_int],
            "llmrs_batch_num_offsets": [c_void_p],
            "llmrs_build_batch": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                  c_void_p, c_int, c_void_p],
            "llmrs_sched_add": [c_void_p, c_void_p, c_int, c_int, c_float, c_int, c_float, c_uint64, c_void_p, c_int],
            "llmrs_sched_check": [c_void_p, c_int, c_int],
            "llmrs_sched_idle": [c_void_p], "llmrs_sched_running": [c_void_p], "llmrs_sched_waiting": [c_void_p],
            "llmrs_sched_plan": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int],
            "llmrs_sched_build": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p],
            "llmrs_sched_commit": [c_void_p, c_void_p, c_int, c_void_p, c_int],
            "llmrs_sched_plan_sources": [c_void_p, c_void_p, c_int], "llmrs_sched_launch": [c_void_p],
            "llmrs_sched_in_flight": [c_void_p], "llmrs_sched_set_max_chunk": [c_void_p, c_int],
            "llmrs_request_info": [c_void_p, c_int, c_void_p],
            "llmrs_request_output": [c_void_p, c_int, c_void_p, c_int],
            "llmrs_request_drop": [c_void_p, c_int],
            "llmrs_request_abort": [c_void_p, c_int],
        }.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = c_int
        lib.llmrs_sched_preemptions.restype = c_longlong
        lib.llmrs_sched_preemptions.argtypes = [c_void_p]
        lib.llmrs_xorshift_next.restype = c_uint64
        lib.llmrs_xorshift_next.argtypes = [POINTER(c_uint64)]
        _configured = True
    return lib


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(c_void_p)


class BatchOffsets:
    """Where each array of a flattened batch starts (in 32-bit words)."""
    __slots__ = ("header", "tokens", "positions", "token_entry", "q_starts", "seq_lens", "slots",
                 "want_rows", "sampling", "slot_maps", "tables", "widths", "words")

    def __init__(self, raw: np.ndarray, n_groups: int, words: int):
        (self.header, self.tokens, self.positions, self.token_entry, self.q_starts, self.seq_lens,
         self.slots, self.want_rows, self.sampling) = (int(x) for x in raw[:9])
        self.slot_maps = [int(raw[9 + 3 * g]) for g in range(n_groups)]
        self.tables = [int(raw[10 + 3 * g]) for g in range(n_groups)]
        self.widths = [int(raw[11 + 3 * g]) for g in range(n_groups)]
        self.words = words


class HostCore:
    """One cache manager + scheduler.  `groups` is a list of (page_size, num_pages, window)."""

    def __init__(self, groups: Sequence[Sequence[int]], max_requests: int, token_budget: int = 2048,
                 max_chunk: int = 0, max_positions: int = 1 << 30):
        self._lib = _lib()
        n = len(groups)
        arr = lambda i: (c_int * max(n, 1))(*[int(g[i]) for g in groups])
        self._h = self._lib.llmrs_core_create(n, arr(0), arr(1), arr(2), max_requests, token_budget, max_chunk, max_positions)
        if not self._h:
            raise CoreError(self._lib.llmrs_create_error().decode())
        self.n_groups = n
        self.groups = [tuple(int(x) for x in g) for g in groups]
        self.max_requests = max_requests
        self._n_off = self._lib.llmrs_batch_num_offsets(self._h)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.llmrs_core_destroy(self._h)
            self._h = None

    def _check(self, rc: int) -> int:
        if rc < 0:
            raise CoreError(self._lib.llmrs_core_error(self._h).decode())
        return rc

    # -- cache manager -----------------------------------------------------
    def acquire_slot(self) -> int:
        return self._check(self._lib.llmrs_slot_acquire(self._h))

    def release_slot(self, slot: int) -> None:
        self._check(self._lib.llmrs_slot_release(self._h, slot))

    def slots_in_use(self) -> int:
        return self._lib.llmrs_slots_in_use(self._h)

    def pages_free(self, g: int = 0) -> int:
        return self._lib.llmrs_pages_free(self._h, g)

    def pages_total(self, g: int = 0) -> int:
        return self._lib.llmrs_pages_total(self._h, g)

    def pages_held(self, slot: int, g: int = 0) -> int:
        return self._check(self._lib.llmrs_pages_held(self._h, slot, g))

    def ensure(self, slot: int, start: int, count: int) -> bool:
        return bool(self._check(self._lib.llmrs_ensure(self._h, slot, start, count)))

    def release_pages(self, slot: int) -> None:
        self._check(self._lib.llmrs_release_pages(self._h, slot))

    def table(self, slot: int, g: int = 0) -> List[int]:
        n = self._check(self._lib.llmrs_table(self._h, slot, g, None, 0))
        out = np.zeros(max(n, 1), dtype=np.int32)
        self._check(self._lib.llmrs_table(self._h, slot, g, _ptr(out), n))
        return out[:n].tolist()

    # -- batch ---------------------------------------------------------------
    def build_batch(self, slots, starts, counts, tokens, want_rows, words: np.ndarray, fixed_widths=None) -> BatchOffsets:
        slots, starts, counts, tokens, want_rows = map(_i32, (slots, starts, counts, tokens, want_rows))
        off = np.zeros(self._n_off, dtype=np.int32)
        fw = _i32(fixed_widths) if fixed_widths is not None else None
        n = self._check(self._lib.llmrs_build_batch(
            self._h, len(slots), _ptr(slots), _ptr(starts), _ptr(counts), _ptr(tokens), _ptr(want_rows),
            len(want_rows), _ptr(fw) if fw is not None else None, _ptr(words), words.size, _ptr(off)))
        return BatchOffsets(off, self.n_groups, n)

    # -- scheduler -----------------------------------------------------------
    def add_request(self, prompt, max_new: int, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0,
                    seed: int = 42, stop=()) -> int:
        """Slot of the request, or -1 when no slot is free right now."""
        prompt, stop = _i32(prompt), _i32(list(stop))
        rc = self._lib.llmrs_sched_add(self._h, _ptr(prompt), len(prompt), max_new, temperature, top_k, top_p,
                                       seed & (2**64 - 1), _ptr(stop), len(stop))
        if rc == -2:
            return -1
        return self._check(rc)

    def check_request(self, n_prompt: int, max_new: int) -> None:
        """Raises what `add_request` would raise for a request that can never run."""
        self._check(self._lib.llmrs_sched_check(self._h, int(n_prompt), int(max_new)))

    def idle(self) -> bool:
        return bool(self._lib.llmrs_sched_idle(self._h))

    def num_running(self) -> int:
        return self._lib.llmrs_sched_running(self._h)

    def num_waiting(self) -> int:
        return self._lib.llmrs_sched_waiting(self._h)

    def preemptions(self) -> int:
        return int(self._lib.llmrs_sched_preemptions(self._h))

    def plan(self):
        """[(slot, start, count, samples)] of the next step."""
        cap = self.max_requests
        a = [np.zeros(cap, dtype=np.int32) for _ in range(4)]
        n = self._check(self._lib.llmrs_sched_plan(self._h, *(_ptr(x) for x in a), cap))
        return [(int(a[0][i]), int(a[1][i]), int(a[2][i]), bool(a[3][i])) for i in range(n)]

    def plan_sources(self) -> List[int]:
        """For each entry of the plan: the row of the step in flight whose sample is the entry's one token, or -1."""
        src = np.zeros(self.max_requests, dtype=np.int32)
        n = self._check(self._lib.llmrs_sched_plan_sources(self._h, _ptr(src), src.size))
        return src[:n].tolist()

    def launch(self) -> None:
        """The planned step has been started: `plan()` may be called for the step after it, before `commit()`
        lands this one."""
        self._check(self._lib.llmrs_sched_launch(self._h))

    def in_flight(self) -> bool:
        return bool(self._lib.llmrs_sched_in_flight(self._h))

    def set_max_chunk(self, max_chunk: int) -> None:
        """The most tokens of one request in a step from now on (0: the step's whole budget)."""
        self._check(self._lib.llmrs_sched_set_max_chunk(self._h, int(max_chunk)))

    def build_planned(self, words: np.ndarray, fixed_widths=None):
        """Flatten the planned step; returns (offsets, n_tokens, n_sampling_rows)."""
        off = np.zeros(self._n_off, dtype=np.int32)
        nt, nw = c_int32(0), c_int32(0)
        fw = _i32(fixed_widths) if fixed_widths is not None else None
        n = self._check(self._lib.llmrs_sched_build(self._h, _ptr(fw) if fw is not None else None, _ptr(words),
                                                    words.size, _ptr(off), ctypes.byref(nt), ctypes.byref(nw)))
        return BatchOffsets(off, self.n_groups, n), nt.value, nw.value

    def commit(self, sampled) -> List[int]:
        sampled = _i32(sampled)
        fin = np.zeros(self.max_requests, dtype=np.int32)
        n = self._check(self._lib.llmrs_sched_commit(self._h, _ptr(sampled), len(sampled), _ptr(fin), fin.size))
        return fin[:n].tolist()

    def request_info(self, slot: int) -> dict:
        info = np.zeros(6, dtype=np.int32)
        self._check(self._lib.llmrs_request_info(self._h, slot, _ptr(info)))
        keys = ("prompt_len", "generated", "computed", "phase", "finish", "preemptions")
        return dict(zip(keys, (int(x) for x in info)))

    def request_output(self, slot: int) -> List[int]:
        n = self._check(self._lib.llmrs_request_output(self._h, slot, None, 0))
        out = np.zeros(max(n, 1), dtype=np.int32)
        self._check(self._lib.llmrs_request_output(self._h, slot, _ptr(out), n))
        return out[:n].tolist()

    def drop_request(self, slot: int) -> None:
        self._check(self._lib.llmrs_request_drop(self._h, slot))

    def abort_request(self, slot: int) -> None:
        """Ends a request wherever it stands; its pages and its slot go back."""
        self._check(self._lib.llmrs_request_abort(self._h, slot))


def xorshift64_stream(seed: int, n: int) -> List[int]:
    """`n` draws of the reference's generator (seed 0 stands for 0xDEADBEEFCAFE)."""
    lib = _lib()
    state = c_uint64(0xDEADBEEFCAFE if seed == 0 else seed)
    return [int(lib.llmrs_xorshift_next(ctypes.byref(state))) for _ in range(n)]
