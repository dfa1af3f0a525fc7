"""Sampling options with the reference's names and meanings
(src/sampler/mod.rs:27-44, src/cli/mod.rs:49-58): temperature 0 is greedy;
top_k 0 (or >= the vocabulary) and top_p >= 1 switch those filters off; each
request draws from a xorshift64 generator of its own, started from `seed`."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int = 42

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError(f"temperature must not be negative, got {self.temperature}")
        if self.top_k < 0:
            raise ValueError(f"top_k must not be negative, got {self.top_k}")
        if not self.top_p > 0:
            raise ValueError(f"top_p must be positive, got {self.top_p}")

    @classmethod
    def reference_defaults(cls) -> "SamplingParams":
        """What the reference's command line samples with when no flag is given."""
        return cls(temperature=0.7, top_k=40, top_p=0.9, seed=42)
