"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.  Matrices and the token table ~ N(0, 0.02^2), norm
weights 1 + N(0, 0.1^2); each tensor has a generator of its own, keyed by the seed
and the tensor's name, so a tensor's values do not depend on which others exist."""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Mapping, Tuple

import torch

from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & (2**63 - 1)


def random_tensors(shapes: Mapping[str, Tuple[int, ...]], kinds: Mapping[str, str], seed: int,
                   dtype=torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    """`kinds[name]` is "matrix" (N(0, 0.02)) or "norm" (1 + N(0, 0.1))."""
    out = {}
    for name, shape in shapes.items():
        g = torch.Generator(device=device)
        g.manual_seed(_tensor_seed(seed, name))
        t = torch.randn(tuple(shape), generator=g, device=device, dtype=torch.float32)
        if kinds[name] == "norm":
            t.mul_(0.1).add_(1.0)
        else:
            t.mul_(0.02)
        out[name] = t.to(dtype)
    return out


def write_model_folder(folder: str, config, tensors: Mapping[str, torch.Tensor]) -> None:
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), dict(tensors), {"format": "pt"})
