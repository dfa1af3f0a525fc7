"""Rotary position encoding(head_dim, rotary_dim, theta, layout, scaling).

freq_i = theta^(-2i/rotary_dim) for pair i (shaders/ops.metal:1030: 1/pow(theta,
2i/head_dim)); the pair is (i, i + rotary_dim/2) in the "split_half" layout that
checkpoints with these tensor names use, or (2i, 2i+1) in the "interleaved" one
the reference's GGUF files need (src/tensor/mod.rs:133-139, src/arch/llama.rs:156).
The reference scales no frequencies; "llama3" scaling is this engine's own:
with wavelength = 2 pi / freq and L = original_max_position_embeddings,
  wavelength < L / high_freq_factor : freq kept
  wavelength > L / low_freq_factor  : freq / factor
  between: s = (L / wavelength - low) / (high - low), freq <- (1 - s) freq / factor + s freq.
The table is made once on the host in double precision and rounded to float32;
the kernel multiplies float(position) by it in 32-bit.
"""
from __future__ import annotations

import math
from typing import Mapping, Optional

import torch

from .base import PositionEncoding, register_position


def rope_inv_freq(rotary_dim: int, theta: float, scaling: Optional[Mapping]) -> torch.Tensor:
    out = []
    for i in range(rotary_dim // 2):
        freq = theta ** (-2.0 * i / rotary_dim)
        if scaling is not None:
            if scaling.get("rope_type", "llama3") != "llama3":
                raise ValueError(f"unsupported rope scaling {scaling.get('rope_type')!r}")
            factor, low, high = float(scaling["factor"]), float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
            orig = float(scaling["original_max_position_embeddings"])
            wavelength = 2.0 * math.pi / freq
            if wavelength > orig / low:
                freq = freq / factor
            elif wavelength >= orig / high:
                s = (orig / wavelength - low) / (high - low)
                freq = (1.0 - s) * freq / factor + s * freq
        out.append(freq)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


class RotaryEncoding(PositionEncoding):
    def __init__(self, params, dtype):
        super().__init__(params, dtype)
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} does not fit head_dim {self.head_dim}")
        layout = params.get("layout", "split_half")
        if layout not in ("split_half", "interleaved"):
            raise ValueError(f"unknown rotary layout {layout!r}")
        self.interleaved = layout == "interleaved"
        self.inv_freq = rope_inv_freq(self.rotary_dim, float(params["theta"]), params.get("scaling"))

    def to(self, device):
        self.inv_freq = self.inv_freq.to(device)

    def rotary(self):
        return self.inv_freq, self.rotary_dim, self.interleaved


register_position("rope", RotaryEncoding)
