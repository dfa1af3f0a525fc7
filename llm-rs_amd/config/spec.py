"""What an architecture hands to the engine: a list of layers made of named
parts, and the order in which they run.

Nothing here knows an architecture.  A `PartSpec` names a registered part kind
(`parts.register_*`) and carries that part's sizes and constants; a `LayerSpec`
names a block arrangement and the parts it is made of: a mixer, a feed-forward
and their norms for the usual arrangements (any of them may be left out where
the arrangement has no use for it), and under `extra` whatever else an
arrangement of another shape needs (norms after a part, a second feed-forward),
each with the family it is built from; a `RunSpec` list says which layer runs
when, so a layer may run twice or read the cache that another run wrote.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    kind: str                       # key in the registry of its family
    prefix: str = ""                # tensor-name prefix, e.g. "model.layers.3.mlp"
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class ExtraPart:
    name: str                       # what the block arrangement calls it, e.g. "post_mixer_norm"
    family: str                     # which registry builds it: "mixer", "feed_forward", "norm", or a family registered with the parts
    spec: PartSpec


@dataclass(frozen=True)
class LayerSpec:
    block: str                      # arrangement, e.g. "prenorm"
    mixer: Optional[PartSpec] = None
    feed_forward: Optional[PartSpec] = None
    mixer_norm: Optional[PartSpec] = None
    feed_forward_norm: Optional[PartSpec] = None
    extra: Tuple[ExtraPart, ...] = ()   # further parts of arrangements that are more than two normed halves


@dataclass(frozen=True)
class RunSpec:
    layer: int                      # index into ModelSpec.layers
    cache_of: Optional[int] = None  # index of an earlier run whose cache this run reads


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    layers: List[LayerSpec]
    schedule: List[RunSpec]
    final_norm: Optional[PartSpec]  # the norm between the last block and the output matrix; None: the stream's rows as they are
    embedding_name: str             # tensor name of the token table
    head_name: Optional[str]        # tensor name of the output matrix; None = tied to the table
    # patterns (fnmatch) of tensor names this architecture's files may hold although the model reads none of them
    ignorable_tensors: Tuple[str, ...] = ()
    embedding_scale: float = 1.0    # the token table's rows are multiplied by this on their way into the stream
    logit_scale: float = 1.0        # logits are multiplied by this, and then,
    logit_softcap: float = 0.0      # if > 0, bent into (-cap, cap): cap * tanh(logit / cap)

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            names = [e.name for e in layer.extra]
            for e in layer.extra:
                if e.name in ("mixer", "feed_forward", "mixer_norm", "feed_forward_norm") or names.count(e.name) > 1:
                    raise ValueError(f"layer {i}: two parts are called {e.name!r}")
        for i, run in enumerate(self.schedule):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"schedule[{i}] names layer {run.layer}, model has {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i:
                    raise ValueError(f"schedule[{i}] reads the cache of run {run.cache_of}, which does not run before it")
                if self.schedule[run.cache_of].cache_of is not None:
                    raise ValueError(f"schedule[{i}] reads the cache of run {run.cache_of}, which owns none")
