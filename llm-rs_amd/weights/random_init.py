"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.  Matrices and the token table ~ N(0, 0.02^2), norm
weights 1 + N(0, 0.1^2); each tensor has a stream of its own, keyed by the seed
and the tensor's name, so a tensor's values do not depend on which others exist.
Element i of a tensor is a function of (its stream's key, i) alone, written once
for the host library and the device kernel (csrc/shared/normal_stream.h): a model
made on the device equals, bit for bit, the one made on the host from the same
seed, so either can be checked against the other's."""
from __future__ import annotations

import hashlib
import json
import os
from collections.abc import Mapping as MappingABC
from typing import Dict, Iterator, Mapping, Tuple

import torch

from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & (2**63 - 1)


def random_tensors(shapes: Mapping[str, Tuple[int, ...]], kinds: Mapping[str, str], seed: int,
                   dtype=torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    """`kinds[name]` is "matrix" (N(0, 0.02)) or "norm" (1 + N(0, 0.1))."""
    if dtype not in (torch.float32, torch.bfloat16):
        raise ValueError(f"random weights are made in float32 or bfloat16, not {dtype}")
    out = {}
    for name, shape in shapes.items():
        mean, std = (1.0, 0.1) if kinds[name] == "norm" else (0.0, 0.02)
        out[name] = fill_normal(torch.empty(tuple(shape), dtype=dtype, device=device), _tensor_seed(seed, name), mean, std)
    return out


class RandomTensors(MappingABC):
    """The same tensors as `random_tensors`, each made when it is asked for and not kept: a model
    that takes them part by part never has a second copy of itself in memory beside the one it
    builds (a 70B shape fills half the device by itself)."""

    def __init__(self, shapes: Mapping[str, Tuple[int, ...]], kinds: Mapping[str, str], seed: int, dtype=torch.bfloat16, device="cpu"):
        self._shapes, self._kinds = dict(shapes), dict(kinds)
        self.seed, self.dtype, self.device = seed, dtype, device

    def shapes(self) -> Dict[str, Tuple[int, ...]]:
        return {n: tuple(s) for n, s in self._shapes.items()}

    def __getitem__(self, name: str) -> torch.Tensor:
        return random_tensors({name: self._shapes[name]}, self._kinds, self.seed, self.dtype, self.device)[name]

    def __iter__(self) -> Iterator[str]:
        return iter(self._shapes)

    def __len__(self) -> int:
        return len(self._shapes)


def fill_normal(t: torch.Tensor, key: int, mean: float, std: float) -> torch.Tensor:
    """t.flat[i] = mean + std * z_i(key), rounded once to t's dtype; by the device kernel for a
    tensor on the GPU, by the host library otherwise: the same bits either way."""
    if t.device.type == "cuda":
        from ..kernels import kernels
        with torch.cuda.device(t.device):
            kernels().fill_normal(t, key, mean, std)
        return t
    import ctypes
    from ..csrc.build import load_host
    lib = load_host()
    fn = lib.llmrs_fill_normal_host
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_float,
                   ctypes.c_float, ctypes.c_int]
    fn.restype = ctypes.c_int
    assert t.is_contiguous()
    if fn(t.data_ptr(), 0 if t.dtype == torch.float32 else 1, t.numel(), key & (2**64 - 1), 0, mean, std, 0) != 0:
        raise RuntimeError("the host library refused to fill the tensor")
    return t


def write_model_folder(folder: str, config, tensors: Mapping[str, torch.Tensor]) -> None:
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), dict(tensors), {"format": "pt"})
