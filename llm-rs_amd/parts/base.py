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


def place(t: torch.Tensor, device, dtype: torch.dtype) -> torch.Tensor:
    """`t` on `device` in `dtype`, contiguous.  The copy to the device is the library's; the
    change of dtype there is this engine's cast kernel."""
    device = torch.device(device)
    if device.type != "cuda" or t.dtype == dtype:
        return t.to(device=device, dtype=dtype).contiguous()
    from ..kernels import kernels
    src = t.to(device=device).contiguous()
    dst = torch.empty(src.shape, dtype=dtype, device=device)
    kernels().cast(dst, src)
    return dst


class TensorSpec(NamedTuple):
    shape: Tuple[int, ...]
    kind: str = "matrix"   # "matrix": N(0, 0.02) in random-weights mode; "norm": 1 + N(0, 0.1)


class Part:
    # True when `forward` only launches kernels whose arguments do not change between steps of
    # the same shape (everything step-specific is read from device memory): such a part may be
    # recorded into a HIP graph.  A part that looks at host values of the step, allocates, or
    # copies between host and device must leave this False; the model is then never recorded.
    graph_safe = False
    # A part whose kernels take something from the host that moves from step to step though the step's sizes stay
    # (a launch shape chosen by how many keys the step sees, say) names here what that choice depends on, any
    # hashable value (parts with equal values are asked once), and says in `recording_key` what it comes to for a
    # step: a recorded step is replayed only for steps with the same key.  None: nothing of the kind.
    recording_signature = None

    def recording_key(self, ctx):
        return ()

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

    def step_weight_bytes(self, seen: set) -> int:
        """Bytes of this part's tensors that a step has to read when it uses each once: every tensor the part
        holds (`seen`: addresses already counted, for tensors that parts share).  A part that reads only some of
        what it holds in a step (the experts a router chose) answers with what a step reads."""
        total = 0
        for v in vars(self).values():
            if isinstance(v, torch.Tensor) and v.data_ptr() not in seen:
                seen.add(v.data_ptr())
                total += v.numel() * v.element_size()
        return total

    def takes_normed_rows(self, ctx, rows: int) -> bool:
        """Whether `forward` may be given `kernels.NormedRows` (rows still to be normed, which the part's
        first product norms itself) in place of the normed input `x`, for a step of `rows` tokens."""
        return False

    def export(self) -> Dict[str, torch.Tensor]:
        """The tensors `load` took, under their names and in the layout of the file they came
        from (whatever `load` fused or reordered is undone), in the dtype the part keeps them in."""
        if not self.tensors():
            return {}
        raise NotImplementedError(f"{type(self).__name__} cannot give its tensors back: it has no export()")


class Norm(Part):
    def forward(self, ctx, h: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        """out[i] = norm(h[rows[i]]) (rows None: every row)."""
        raise NotImplementedError

    def deferred_weight(self) -> Optional[torch.Tensor]:
        """For a norm of the form x / rms(x) * weight: the float32 weight, which lets the product before it
        prepare its rows and the product after it finish them (`kernels.NextNorm`, `kernels.NormedRows`);
        None for any other norm."""
        return None

    def deferred_eps(self) -> Optional[float]:
        """For a norm of that form: its eps, which lets a product that sees whole rows finish the norm itself
        (`kernels.NextNorm` with eps); None for any other norm."""
        return None

    def deferred(self, ctx, h: torch.Tensor):
        """The norm of every row of `h`, not computed here: a `kernels.NormedRows` for a part that
        `takes_normed_rows`, or the normed rows themselves (a tensor) where the last product that added into `h`
        finished this norm, or None when neither holds (then `forward` runs)."""
        return None


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
    """An arrangement of parts around the residual stream.  It gets the layer's parts by the
    names the `LayerSpec` gives them: "mixer", "feed_forward", "mixer_norm",
    "feed_forward_norm" and whatever the spec lists under `extra`; `needs` names those an
    arrangement cannot do without.  The layer's cache belongs to the part called "mixer"."""

    needs = ("mixer",)

    # True only for an arrangement that vouches for this: when its `forward` returns, whatever
    # `ctx.left_for(h)` gives describes `h` as it stands (the last thing that touched `h` was a part's
    # `forward`, and what an earlier product left was dropped before that part ran).  The model drops
    # it after any block that does not say so.
    keeps_left_current = False

    def first_norm(self) -> Optional[Norm]:
        """The norm that reads the stream first when this block runs, if the block before may prepare it."""
        return None

    def __init__(self, named: Mapping[str, Part]):
        missing = [n for n in self.needs if named.get(n) is None]
        if missing:
            raise ValueError(f"block arrangement {type(self).__name__} needs the parts {', '.join(missing)}")
        self.named: Dict[str, Part] = {n: p for n, p in named.items() if p is not None}
        self.mixer: Optional[Mixer] = self.named.get("mixer")
        self.feed_forward: Optional[FeedForward] = self.named.get("feed_forward")
        self.mixer_norm: Optional[Norm] = self.named.get("mixer_norm")
        self.feed_forward_norm: Optional[Norm] = self.named.get("feed_forward_norm")

    def parts(self):
        return tuple(self.named.values())

    def cache_need(self):
        """What the layer asks of the cache manager: its mixer's need, or nothing."""
        return None if self.mixer is None else self.mixer.cache_need()

    @staticmethod
    def normed_input(ctx, h: torch.Tensor, norm: "Norm", part: Part, then: Optional["Norm"]):
        """The input of `part`: norm(h), computed here, or left to the part's first product where the norm can be
        deferred and the part takes such rows (a step of few tokens whose stream was last written by a product
        that prepared this norm: then no norm kernel runs).  `then` is the norm that reads the stream after `part`."""
        rows = norm.deferred(ctx, h)
        if not isinstance(rows, torch.Tensor) and not part.takes_normed_rows(ctx, h.shape[0]):
            rows = None         # (rows already normed are any part's input; rows still to be scaled only the parts' that can)
        # The part is about to change the stream: what was left stops describing it now.  (The rows handed over
        # keep their own references; a part that leaves something for `then` notes it when it is done.)
        ctx.note_left(h, None)
        ctx.upcoming_norm = then
        if rows is not None:
            return rows
        x = ctx.workspace("block.x", (h.shape[0], h.shape[1]), part.dtype)
        norm.forward(ctx, h, x)
        return x

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


# Families of parts that a layer's `extra` list may name: family -> the table of its kinds.  The three below are
# what the four usual places of a layer are built from; an arrangement that needs parts of another nature (a router
# shared by two feed-forwards, a gate) registers a family for them.
FAMILIES: Dict[str, Dict[str, Callable]] = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS}


def register_part_family(family: str) -> Callable:
    """Makes `family` a family of parts that `LayerSpec.extra` may name; returns the function that registers its
    kinds, `register(kind, factory)` with `factory(spec, dtype)` as for the other families."""
    table = FAMILIES.setdefault(family, {})
    return _register(table, family)


def build_part(family: str, spec: PartSpec, dtype) -> Part:
    if family not in FAMILIES:
        raise KeyError(f"unknown family of parts {family!r} (registered: {', '.join(sorted(FAMILIES))})")
    return _build(FAMILIES[family], family, spec.kind, spec, dtype)


def build_block(layer_spec, dtype) -> Block:
    opt = lambda build, spec: None if spec is None else build(spec, dtype)
    named = {"mixer_norm": opt(build_norm, layer_spec.mixer_norm), "mixer": opt(build_mixer, layer_spec.mixer),
             "feed_forward_norm": opt(build_norm, layer_spec.feed_forward_norm),
             "feed_forward": opt(build_feed_forward, layer_spec.feed_forward)}
    for extra in layer_spec.extra:
        named[extra.name] = build_part(extra.family, extra.spec, dtype)
    return _build(BLOCKS, "block arrangement", layer_spec.block, named)
