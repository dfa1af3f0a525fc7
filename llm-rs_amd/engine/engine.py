"""The engine: configuration -> model -> cache -> step function -> scheduler ->
sampler.  `submit()` and `advance()` are the reference's serving loop without the
HTTP channel (src/serve/engine.rs:161-231): requests come in at any time, a call
of `advance()` plans, flattens, runs, samples, commits and frees what finished, and
says which request got which token.  `generate()` is that loop for a list of prompts."""
from __future__ import annotations

import gc
import sys
import time
from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Sequence, Union

import numpy as np
import torch

from ..cache import CacheManager, CoreError, cache_kind
from ..config import load_config
from ..sampling import Sampler, SamplingParams
from ..weights import RandomTensors, load_tensors, random_tensors
from .model import Model
from .step import StepEntry, StepRunner

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32,
           "fp32": torch.float32, torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    generated_tokens: int = 0
    steps: int = 0
    seconds: float = 0.0
    preemptions: int = 0
    first_token_seconds: float = 0.0
    device_seconds: float = 0.0          # device time of the steps, when the engine was asked to measure it
    first_token_device_seconds: float = 0.0


@dataclass
class Finished:
    tokens: List[int]
    reason: str          # "stop" or "length"


@dataclass
class Emitted:
    """What one step gave one request: a token (none when a stop token ended it: that token is
    not part of the output) and, if the request is finished, why ("stop" or "length")."""
    request: int
    token: Optional[int]
    finished: Optional[str] = None


@dataclass
class _Flight:
    """A step that was started and whose samples the scheduler has not been told."""
    owners: List[tuple]              # (slot, request) of the entries that sample, in their order
    ids: Optional[torch.Tensor]      # their samples on the device (the sampler's buffer: good until the next step samples)
    host: Optional[torch.Tensor]     # the same on their way to the host
    landed: object                   # an event behind that copy, or None where copies are synchronous
    events: Optional[tuple]          # (before the first kernel, after sampling) when device time is measured


@dataclass
class _Submitted:
    prompt: Sequence[int]
    limit: int
    params: SamplingParams
    stop: Sequence[int]


class Engine:
    def __init__(self, config, tensors: Mapping[str, torch.Tensor], *, dtype="bfloat16", device="cuda",
                 page_size: int = 16, num_pages=None, kv_memory_fraction: float = 0.8, max_requests: int = 256,
                 max_batch_tokens: int = 2048, max_chunk: int = 0, max_seq_len: Optional[int] = None, log: bool = False,
                 overlap: bool = True):
        """`overlap`: `advance()` starts a step before the samples of the step before it have reached the host (the
        device hands them over), so that the device does not wait while the host reads samples and plans; outputs
        are the same.  Without it a step is planned only when the one before has been read."""
        if dtype not in _DTYPES:
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype!r}")
        self.config = config
        self.dtype = _DTYPES[dtype]
        self.device = torch.device(device)
        self.log = log
        if self.device.type == "cuda":
            from ..kernels import kernels
            kernels()    # no GPU or no kernel library: fail here, with that message, before any weight moves
        spec = config.model_spec()
        self.model = Model(spec, self.dtype, self.device)
        self.model.load(tensors)
        self.max_seq_len = min(max_seq_len or spec.max_positions, spec.max_positions)
        needs = self.model.cache_needs()
        if num_pages is None:
            num_pages = self._pages_from_memory(needs, page_size, kv_memory_fraction, max_requests, max_chunk or max_batch_tokens)
        self.cache = CacheManager(needs, self.dtype, self.device, page_size, num_pages, max_requests,
                                  token_budget=max_batch_tokens, max_chunk=max_chunk, max_positions=self.max_seq_len)
        self.runner = StepRunner(self.model, self.cache, self.device)
        self.sampler = Sampler(self.device)
        self.max_batch_tokens = max_batch_tokens
        self.last_stats = GenerationStats()
        self._next_request = 0
        self._waiting: Dict[int, _Submitted] = {}          # submitted, no slot yet (in order of submission)
        self._request_of: Dict[int, int] = {}              # slot -> request, for those the scheduler holds
        self._samples_randomly: set = set()                 # of those, the slots that do not decode greedily
        self.overlap = bool(overlap)
        self._flight: Optional[_Flight] = None               # the step in flight (overlap)
        self._ids_host = [None, None]                        # pinned room for samples on their way to the host, in turns
        self._ids_turn = 0
        self._steps = 0
        self._step_events: List[tuple] = []                 # (before the first kernel, after sampling) of measured steps
        # A full collection now, while nothing waits for it: building the model has made so many
        # objects that the collector would otherwise choose a moment among the first decode steps to
        # walk everything the libraries hold (measured: one pause of 40 ms there).
        gc.collect()
        if log:
            for g, grp in enumerate(self.cache.groups):
                gb = grp.num_pages * page_size * grp.bytes_per_token() / 1e9
                print(f"KV pool {g}: {grp.num_pages} pages x {page_size} tokens = {grp.num_pages * page_size} max tokens, {gb:.2f} GB",
                      file=sys.stderr)

    # -- construction ----------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, **kw) -> "Engine":
        config = load_config(folder)
        dtype = kw.get("dtype", "bfloat16")
        if dtype not in _DTYPES:
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype!r}")
        if torch.device(kw.get("device", "cuda")).type == "cuda":
            from ..kernels import kernels
            kernels()    # no GPU or no kernel library: say so before the first tensor is read
        spec = config.model_spec()
        probe = Model(spec, torch.bfloat16, "cpu")
        want = {n: t.shape for n, t in probe.tensors().items()}
        tensors = load_tensors(folder, want, device="cpu", log=kw.get("log", False), compute=_DTYPES[dtype],
                               ignorable=spec.ignorable_tensors)
        return cls(config, tensors, **kw)

    @classmethod
    def from_random(cls, config, seed: int, **kw) -> "Engine":
        """Random weights made where the engine lives, without a folder in between, each tensor when
        the model takes it: the same values as `random_model_tensors(config, seed)` gives on the host."""
        probe = Model(config.model_spec(), torch.bfloat16, "cpu")
        specs = probe.tensors()
        tensors = RandomTensors({n: s.shape for n, s in specs.items()}, {n: s.kind for n, s in specs.items()}, seed,
                                dtype=torch.bfloat16, device=kw.get("device", "cuda"))
        return cls(config, tensors, **kw)

    def weights(self) -> Dict[str, torch.Tensor]:
        """The model's tensors on the host, by file name and in the file's layout (`Model.weights`)."""
        return self.model.weights()

    def _pages_from_memory(self, needs, page_size, fraction, max_requests, max_step_tokens):
        """Pages that fit `fraction` of the memory still free after the weights and after what every request
        slot gets of fixed size; what a token and a slot cost is the cache kinds' to say."""
        if self.device.type != "cuda":
            if any(need is not None and cache_kind(need).paged for need, _ in needs):
                raise ValueError("num_pages must be given when the engine is not on a GPU")
            return []
        free, _ = torch.cuda.mem_get_info(self.device)
        return CacheManager.pages_that_fit(needs, self.dtype, page_size, free, fraction, max_requests, self.max_seq_len,
                                           max_step_tokens)

    # -- manual stepping (trace replay, tests) -----------------------------------
    def open_request(self) -> int:
        """A slot for a request that the caller steps by hand."""
        return self.cache.core.acquire_slot()

    def close_request(self, slot: int) -> None:
        self.cache.core.release_slot(slot)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        return self.runner.run(entries)

    # -- requests that come and go -----------------------------------------------------
    def submit(self, prompt: Sequence[int], max_new_tokens: int = 256, temperature: float = 0.0, top_k: int = 0,
               top_p: float = 1.0, seed: int = 42, stop_token_ids: Sequence[int] = ()) -> int:
        """Hands a request to the scheduler; returns its number.  It joins the batch at the next
        `advance()` that has a slot and pages for it.  Every request has its own generator started
        from `seed`, so its output does not depend on what it is batched with."""
        vocab = self.model.spec.vocab_size
        if len(prompt) == 0:
            raise ValueError("the prompt is empty")
        if min(prompt) < 0 or max(prompt) >= vocab:
            raise ValueError(f"token ids must be in [0, {vocab})")
        if max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        # A request that could never run (longer than the positions allow, more pages at once than a
        # pool has) is refused here, not at some later advance(), where it would stand in the way
        # of every request behind it.
        try:
            self.cache.core.check_request(len(prompt), int(max_new_tokens))
        except CoreError as e:
            raise ValueError(str(e)) from None
        request = self._next_request
        self._next_request += 1
        self._waiting[request] = _Submitted(list(prompt), int(max_new_tokens),
                                            SamplingParams(temperature, top_k, top_p, seed), list(stop_token_ids))
        return request

    def measure_device_time(self, on: bool = True) -> None:
        """From now on every step of `advance()` is bracketed by two events on the device, and
        `device_seconds()` says how long the device worked (the reference's gpu= figure, src/main.rs:141-150)."""
        self.runner.time_device = bool(on)
        self._step_events = []

    def device_seconds(self) -> float:
        """Device time of the steps since the last call (waits for the device)."""
        if not self._step_events:
            return 0.0
        torch.cuda.synchronize(self.device)
        total = sum(a.elapsed_time(b) for a, b in self._step_events) * 1e-3
        self._step_events = []
        return total

    def has_unfinished(self) -> bool:
        return bool(self._waiting) or bool(self._request_of) or self._flight is not None

    def cancel(self, request: int) -> None:
        """Ends a request wherever it stands; its pages and its slot go back."""
        if self._waiting.pop(request, None) is not None:
            return
        for slot, r in list(self._request_of.items()):
            if r == request:
                self.cache.core.abort_request(slot)
                self._forget(slot)

    def _forget(self, slot: int) -> None:
        self._request_of.pop(slot)
        self._samples_randomly.discard(slot)

    def _admit(self) -> None:
        core = self.cache.core
        for request in list(self._waiting):
            sub = self._waiting[request]
            slot = core.add_request(sub.prompt, sub.limit, sub.params.temperature, sub.params.top_k, sub.params.top_p,
                                    sub.params.seed, sub.stop)
            if slot < 0:                # no slot free right now: this one and those behind it wait
                return
            del self._waiting[request]
            self._request_of[slot] = request
            if sub.params.temperature != 0.0:
                self._samples_randomly.add(slot)

    def _start_step(self, after: Optional[_Flight]) -> Optional[_Flight]:
        """Plans a step and starts it on the device, sampling included, without waiting for anything.  `after`: the
        step in flight whose samples this one's tokens may be.  None when nothing could be planned."""
        logits, n_want, plan = self.runner.run_planned(after.ids if after is not None else None)
        if not plan:
            return None
        ids = host = landed = events = None
        if n_want:
            ids = self.sampler.sample(logits, self.runner.ctx.sampling, not self._samples_randomly)
        if self.runner.time_device and self.runner.started is not None:
            done = torch.cuda.Event(enable_timing=True)
            done.record()
            events = (self.runner.started, done)
        if n_want:
            if self.device.type == "cuda":
                self._ids_turn ^= 1
                host = self._ids_host[self._ids_turn]
                if host is None or host.numel() < n_want:
                    host = self._ids_host[self._ids_turn] = torch.zeros(max(2 * n_want, 256), dtype=torch.int32, pin_memory=True)
                host = host[:n_want]
                host.copy_(ids, non_blocking=True)
                landed = torch.cuda.Event()
                landed.record()
            else:
                host = ids.clone()
        self._steps += 1
        return _Flight([(p[0], self._request_of[p[0]]) for p in plan if p[3]], ids, host, landed, events)

    def _land_step(self, flight: _Flight) -> List[Emitted]:
        """Waits for a started step's samples, tells the scheduler, and returns what each sampling request got."""
        core = self.cache.core
        if flight.events is not None:
            self._step_events.append(flight.events)
        sampled = []
        if flight.host is not None:
            if flight.landed is not None:
                flight.landed.synchronize()
            sampled = flight.host.numpy().copy()
            # A sampler or hand-over fault must not go on as "the request decodes from token 0": fail here.
            vocab = self.model.spec.vocab_size
            if len(sampled) and (int(sampled.min()) < 0 or int(sampled.max()) >= vocab):
                raise RuntimeError(f"a step sampled token ids outside [0, {vocab}): {int(sampled.min())}..{int(sampled.max())}")
        finished = set(core.commit(sampled))
        out: List[Emitted] = []
        for (slot, request), token in zip(flight.owners, sampled):
            if self._request_of.get(slot) != request:
                continue                    # it ended while this step was in flight (a stop token, a cancel): dropped
            if slot in finished:
                reason = "stop" if core.request_info(slot)["finish"] == 1 else "length"
                out.append(Emitted(request, None if reason == "stop" else int(token), reason))
                core.drop_request(slot)
                self._forget(slot)
            else:
                out.append(Emitted(request, int(token)))
        return out

    def _advance_overlapped(self) -> List[Emitted]:
        core = self.cache.core
        self._admit()
        if self._flight is None:
            if core.idle():
                return []
            self._flight = self._start_step(None)
            if self._flight is None:
                raise RuntimeError("the scheduler planned nothing although requests are waiting")
            core.launch()
        # the step after it, before this one's samples are known (nothing, when all it could run waits for pages
        # or for those samples: then the next call starts afresh)
        landing, ahead = self._flight, self._start_step(self._flight)
        try:
            out = self._land_step(landing)
        finally:
            # Whatever happens while the first step lands (an interrupt included), engine and scheduler go on
            # agreeing about which step is in flight: the one that was started ahead, once the scheduler has
            # taken the landed one (commit), or still the first one if it has not.
            if not core.in_flight():
                self._flight = ahead
                if ahead is not None:
                    core.launch()
        self._admit()
        return out

    def advance(self) -> List[Emitted]:
        """One step of the scheduler: admits what fits, runs the planned batch (prompt portions
        beside decoded tokens), samples, and returns what each sampling request got.  Requests
        still inside their prompts get nothing in that step.  (With `overlap` what is returned is
        the step before the one this call started; the last calls only collect.)"""
        if self.overlap:
            return self._advance_overlapped()
        self._admit()
        if self.cache.core.idle():
            return []
        step = self._start_step(None)                # in turn: a step is started, and read before anything else happens
        if step is None:
            raise RuntimeError("the scheduler planned nothing although requests are waiting")
        out = self._land_step(step)
        self._admit()
        return out

    # -- generation ----------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: Union[int, Sequence[int]] = 256, temperature: float = 0.0,
                 top_k: int = 0, top_p: float = 1.0, seed: Union[int, Sequence[int]] = 42,
                 stop_token_ids: Sequence[int] = (), return_reasons: bool = False):
        """Token ids generated for each prompt.  Every request has its own generator
        started from `seed` (one for all, or one each), so a prompt's output does not
        depend on what it was batched with.  `max_new_tokens` too is one for all or one each
        (a request of the reference carries its own max_tokens, serve/engine.rs:24,35)."""
        n = len(prompts)
        seeds = [seed] * n if isinstance(seed, int) else list(seed)
        if len(seeds) != n:
            raise ValueError("one seed, or one for each prompt")
        limits = [max_new_tokens] * n if isinstance(max_new_tokens, int) else [int(m) for m in max_new_tokens]
        if len(limits) != n:
            raise ValueError("one max_new_tokens, or one for each prompt")
        if self.has_unfinished():
            raise RuntimeError("generate() needs the engine to itself: requests submitted earlier are still running")
        vocab = self.model.spec.vocab_size
        for i, p in enumerate(prompts):
            if len(p) == 0:
                raise ValueError(f"prompt {i} is empty")
            if min(p) < 0 or max(p) >= vocab:
                raise ValueError(f"prompt {i}: token ids must be in [0, {vocab})")
        results: List[Optional[Finished]] = [None] * n
        stats = GenerationStats(prompt_tokens=sum(len(p) for p in prompts))
        t0 = time.perf_counter()
        steps0, preempt0 = self._steps, self.cache.core.preemptions()
        index_of: Dict[int, int] = {}
        tokens: Dict[int, List[int]] = {}
        try:
            for i, p in enumerate(prompts):
                if limits[i] <= 0:              # nothing to generate: done before it starts
                    results[i] = Finished([], "length")
                    continue
                r = self.submit(p, limits[i], temperature, top_k, top_p, seeds[i], stop_token_ids)
                index_of[r], tokens[r] = i, []
            while self.has_unfinished():
                for e in self.advance():
                    if stats.first_token_seconds == 0.0:
                        stats.first_token_seconds = time.perf_counter() - t0
                        stats.first_token_device_seconds = self.device_seconds()
                    if e.token is not None:
                        tokens[e.request].append(e.token)
                    if e.finished:
                        results[index_of[e.request]] = Finished(tokens.pop(e.request), e.finished)
        except BaseException:
            for r in index_of:                  # leave the engine as it was found
                self.cancel(r)
            flight, self._flight = self._flight, None
            if flight is not None and self.cache.core.in_flight():
                # (every entry of the step in flight is dead now: its samples are dropped)
                self.cache.core.commit([0] * len(flight.owners))
            raise
        if self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        stats.seconds = time.perf_counter() - t0
        stats.device_seconds = stats.first_token_device_seconds + self.device_seconds()
        stats.steps = self._steps - steps0
        stats.generated_tokens = sum(len(r.tokens) for r in results)
        stats.preemptions = self.cache.core.preemptions() - preempt0
        self.last_stats = stats
        return results if return_reasons else [r.tokens for r in results]


def random_model_tensors(config, seed: int, dtype=torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    """The tensors a configuration's model needs, drawn from `seed`."""
    probe = Model(config.model_spec(), torch.bfloat16, "cpu")
    specs = probe.tensors()
    return random_tensors({n: s.shape for n, s in specs.items()}, {n: s.kind for n, s in specs.items()},
                          seed, dtype=dtype, device=device)
