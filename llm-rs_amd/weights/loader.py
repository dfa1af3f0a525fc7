"""Weights by tensor name from a model folder, with one error that names every
missing, unexpected and mis-shaped tensor.  The reference looks tensors up by
name and panics on the first missing one, without a shape check
(src/arch/mod.rs:52-61, src/arch/llama.rs:80-94); like it, this loader leaves
alone what an architecture says its files may carry without the model using it
(a stored table of rotation frequencies, the output matrix of a tied model):
such names are reported in a line on stderr, not as an error."""
from __future__ import annotations

import fnmatch
import json
import os
import sys
import time
from typing import Dict, Iterable, List, Mapping, Sequence, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightError(ValueError):
    """`missing`, `unexpected` and `wrong_shape` hold what the message lists."""

    def __init__(self, missing, unexpected, wrong_shape, where=""):
        self.missing, self.unexpected, self.wrong_shape = list(missing), list(unexpected), list(wrong_shape)
        lines = [f"weights do not fit the model{' (' + where + ')' if where else ''}:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name}: expected {list(want)} got {list(got)}")
        super().__init__("\n".join(lines))


def stored_dtype(dtype: torch.dtype, compute: torch.dtype = torch.bfloat16) -> torch.dtype:
    """How a tensor is kept: bfloat16, except that integer tables become int32 and
    what the file stores in 32-bit (or wider) floating point stays float32.  A
    float16 file read for an engine that computes in float32 is widened, not
    rounded to bfloat16's eight bits: the 32-bit path sees the file's own values
    (the reference picks its kernel by the tensor's own dtype,
    src/backend/metal/mod.rs:503-512)."""
    if dtype in (torch.float32, torch.float64):
        return torch.float32
    if dtype == torch.float16 and compute == torch.float32:
        return torch.float32
    if dtype.is_floating_point:
        return torch.bfloat16
    return torch.int32


def check_tensors(have: Mapping[str, Tuple[int, ...]], want: Mapping[str, Tuple[int, ...]], where: str = "",
                  ignorable: Sequence[str] = ()) -> List[str]:
    """Raises one WeightError for everything that does not fit.  Names in `have` that the model does
    not use are unexpected, unless they match one of the `ignorable` patterns: those are returned
    (and said on stderr), the model just does not read them."""
    missing = [n for n in want if n not in have]
    extra = [n for n in have if n not in want]
    ignored = sorted(n for n in extra if any(fnmatch.fnmatchcase(n, pat) for pat in ignorable))
    unexpected = [n for n in extra if n not in ignored]
    wrong = [(n, tuple(want[n]), tuple(have[n])) for n in want if n in have and tuple(have[n]) != tuple(want[n])]
    if missing or unexpected or wrong:
        raise WeightError(sorted(missing), sorted(unexpected), wrong, where)
    if ignored:
        shown = ", ".join(ignored[:4]) + (f", ... ({len(ignored)} in all)" if len(ignored) > 4 else "")
        print(f"Warning: tensors the model does not use are left unread{' (' + where + ')' if where else ''}: {shown}", file=sys.stderr)
    return ignored


def open_model_files(folder: str) -> Dict[str, SafetensorsFile]:
    """name -> the file that holds it; one model.safetensors or the shards of an index."""
    index = os.path.join(folder, "model.safetensors.index.json")
    single = os.path.join(folder, "model.safetensors")
    files: Dict[str, SafetensorsFile] = {}
    where: Dict[str, SafetensorsFile] = {}
    if os.path.exists(index):
        with open(index) as f:
            weight_map = json.load(f)["weight_map"]
        for name, shard in weight_map.items():
            if shard not in files:
                files[shard] = SafetensorsFile(os.path.join(folder, shard))
            if name in files[shard].entries:
                where[name] = files[shard]
        return where
    if not os.path.exists(single):
        raise SafetensorsError(f"no model.safetensors in {folder}")
    f = SafetensorsFile(single)
    return {name: f for name in f.names()}


def load_tensors(folder: str, want: Mapping[str, Tuple[int, ...]], device="cpu", log=True,
                 compute: torch.dtype = torch.bfloat16, ignorable: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """Read the tensors `want` names (name -> shape) from `folder`, check them all
    before the first copy, and bring them to `device` in their kept dtype (which
    depends on the dtype the engine computes in, see `stored_dtype`)."""
    start = time.time()
    where = open_model_files(folder)
    check_tensors({n: f.entries[n][1] for n, f in where.items()}, want, folder, ignorable)
    out: Dict[str, torch.Tensor] = {}
    nbytes = 0
    for name in want:
        t = where[name].tensor(name)
        nbytes += t.numel() * t.dtype.itemsize
        out[name] = t.to(device=device, dtype=stored_dtype(t.dtype, compute))
    if log:
        dt = max(time.time() - start, 1e-9)
        print(f"Loaded model weights: {nbytes / 2**30:.2f} GB in {dt:.3f}s ({nbytes / 2**30 / dt:.1f} GB/s)", file=sys.stderr)
    return out
