"""Interfaces of the parts a layer is put together from, and their registries.

A part gets its sizes and constants from a `PartSpec` and the activation dtype;
it names the tensors it needs (`tensors()`), takes them (`load()`) and runs on a
step's tokens (`forward()`).  No part knows which model it is in: everything
about the step comes through the `StepContext`, everything about its memory
through the `CacheView` the engine hands it.

Conventions of `forward`:
  * the residual stream `h` is float32 [T, hidden]; a mixer or feed-forward ADDS
    its result into `h` (the sum is 32-bit; the kernels fuse it into the last
    product's epilogue);
  * `x` is the normed input in the activation dtype, [T, hidden];
  * a norm reads float32 rows and writes the activation dtype.
"""
from __future__ import annotations

from typing import Callable, Dict, Mapping, NamedTuple, Optional, Tuple

import torch

from ..config.spec import PartSpec


class TensorSpec(NamedTuple):
    shape: Tuple[int, ...]
    kind: str = "matrix"   # "matrix": N(0, 0.02) in random-weights mode; "norm": 1 + N(0, 0.1)


class Part:
    # True when `forward` only launches kernels whose arguments do not change between steps of
    # the same shape (everything step-specific is read from device memory): such a part may be
    # recorded into a HIP graph.  A part that looks at host values of the step, allocates, or
    # copies between host and device must leave this False; the model is then never recorded.
    graph_safe = False

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        self.spec = spec
        self.prefix = spec.prefix
        self.dtype = dtype

    def name(self, leaf: str) -> str:
        return f"{self.prefix}.{leaf}" if self.prefix else leaf

    def tensors(self) -> Dict[str, TensorSpec]:
        """Full tensor name -> shape and kind, of everything `load` will ask for."""
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor], device) -> None:
        pass


class Norm(Part):
    def forward(self, ctx, h: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        """out[i] = norm(h[rows[i]]) (rows None: every row)."""
        raise NotImplementedError


class PositionEncoding:
    """How positions enter a mixer.  `rotary()` returns (inv_freq table, rotary_dim,
    interleaved) when the encoding is a rotation the attention kernels fuse, else
    None, and then `apply(ctx, q, k)` changes q and k [T, heads, head_dim] in place."""

    def __init__(self, params: Mapping, dtype: torch.dtype):
        self.params = dict(params)

    def to(self, device) -> None:
        pass

    def rotary(self):
        return None

    def apply(self, ctx, q: torch.Tensor, k: Optional[torch.Tensor]) -> None:
        pass


class Mixer(Part):
    def cache_need(self):
        """A `cache.PagedKV`, a `cache.FixedState`, or None."""
        return None

    def forward(self, ctx, x: torch.Tensor, h: torch.Tensor, cache) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, x: torch.Tensor, h: torch.Tensor) -> None:
        raise NotImplementedError


class Block:
    """An arrangement of a mixer, a feed-forward and their norms around the residual stream."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, feed_forward_norm: Norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def parts(self):
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def forward(self, ctx, h: torch.Tensor, cache) -> None:
        raise NotImplementedError


MIXERS: Dict[str, Callable] = {}
FEED_FORWARDS: Dict[str, Callable] = {}
NORMS: Dict[str, Callable] = {}
POSITIONS: Dict[str, Callable] = {}
BLOCKS: Dict[str, Callable] = {}


def _register(table: Dict[str, Callable], family: str):
    def register(kind: str, factory: Callable) -> None:
        table[kind] = factory
    register.__doc__ = f"Make `kind` available as a {family}; `factory(spec_or_params, dtype)` builds it."
    return register


register_mixer = _register(MIXERS, "mixer")
register_feed_forward = _register(FEED_FORWARDS, "feed-forward")
register_norm = _register(NORMS, "norm")
register_position = _register(POSITIONS, "position encoding")
register_block = _register(BLOCKS, "block arrangement")


def _build(table: Dict[str, Callable], family: str, kind: str, *args):
    if kind not in table:
        raise KeyError(f"unknown {family} kind {kind!r} (registered: {', '.join(sorted(table))})")
    return table[kind](*args)


def build_mixer(spec: PartSpec, dtype) -> Mixer:
    return _build(MIXERS, "mixer", spec.kind, spec, dtype)


def build_feed_forward(spec: PartSpec, dtype) -> FeedForward:
    return _build(FEED_FORWARDS, "feed-forward", spec.kind, spec, dtype)


def build_norm(spec: PartSpec, dtype) -> Norm:
    return _build(NORMS, "norm", spec.kind, spec, dtype)


def build_position(params: Optional[Mapping], dtype) -> Optional[PositionEncoding]:
    if params is None:
        return None
    return _build(POSITIONS, "position encoding", params["kind"], params, dtype)


def build_block(layer_spec, dtype) -> Block:
    return _build(BLOCKS, "block arrangement", layer_spec.block,
                  build_mixer(layer_spec.mixer, dtype), build_feed_forward(layer_spec.feed_forward, dtype),
                  build_norm(layer_spec.mixer_norm, dtype), build_norm(layer_spec.feed_forward_norm, dtype))
