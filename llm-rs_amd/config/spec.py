"""What an architecture hands to the engine: a list of layers made of named
parts, and the order in which they run.

Nothing here knows an architecture.  A `PartSpec` names a registered part kind
(`parts.register_*`) and carries that part's sizes and constants; a `LayerSpec`
puts a mixer, a feed-forward and their norms into a block arrangement; a
`RunSpec` list says which layer runs when, so a layer may run twice or read the
cache that another run wrote.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    kind: str                       # key in the registry of its family
    prefix: str = ""                # tensor-name prefix, e.g. "model.layers.3.mlp"
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    block: str                      # arrangement, e.g. "prenorm"
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec


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
    final_norm: PartSpec
    embedding_name: str             # tensor name of the token table
    head_name: Optional[str]        # tensor name of the output matrix; None = tied to the table

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        for i, run in enumerate(self.schedule):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"schedule[{i}] names layer {run.layer}, model has {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i:
                    raise ValueError(f"schedule[{i}] reads the cache of run {run.cache_of}, which does not run before it")
                if self.schedule[run.cache_of].cache_of is not None:
                    raise ValueError(f"schedule[{i}] reads the cache of run {run.cache_of}, which owns none")
