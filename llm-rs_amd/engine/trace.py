"""Trace replay: given token ids go through the engine's own model, step function,
cache and kernels step by step, and the logits at the asked places come back.
Nothing is sampled.  It is the pair of loops that feed tokens through `forward`
in the reference (src/main.rs:102-139, src/serve/engine.rs:189-196) with the
choice of what runs when taken from a trace instead of a scheduler."""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, Optional

import numpy as np
import torch

from .engine import Engine
from .step import StepEntry

TRACE_ROUND_TO = 64      # a request's tokens count towards --max-tokens rounded up to this


class TraceReplayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16, device: str = "cuda",
                 max_requests: int = 64):
        if TRACE_ROUND_TO % page_size:
            raise ValueError(f"page_size {page_size} must divide {TRACE_ROUND_TO}")
        num_pages = max(-(-max_tokens // page_size), 1)
        self._bind(Engine.from_folder(model_dir, dtype=dtype, device=device, page_size=page_size,
                                      num_pages=num_pages, max_requests=max_requests))

    @classmethod
    def for_engine(cls, engine: Engine) -> "TraceReplayer":
        """Replays traces through an engine that exists already (one made from random weights, say)."""
        self = cls.__new__(cls)
        self._bind(engine)
        return self

    def _bind(self, engine: Engine) -> None:
        self.engine = engine
        self.slot: Dict[str, int] = {}
        self.position: Dict[str, int] = {}

    def step(self, record: dict) -> Optional[np.ndarray]:
        """Runs one step of the trace; returns float32 [wanted, vocab] or None."""
        entries = []
        for e in record.get("entries", []):
            rid = str(e["id"])
            tokens = [int(t) for t in e["tokens"]]
            if not tokens:
                continue
            if rid not in self.slot:
                self.slot[rid] = self.engine.open_request()
                self.position[rid] = 0
            entries.append(StepEntry(self.slot[rid], self.position[rid], tokens, [int(w) for w in e.get("want", [])]))
            self.position[rid] += len(tokens)
        logits = self.engine.step(entries) if entries else None
        out = None if logits is None else logits.detach().cpu().numpy().astype("<f4", copy=False)
        for rid in record.get("end", []):
            rid = str(rid)
            if rid in self.slot:
                self.engine.close_request(self.slot.pop(rid))
                self.position.pop(rid)
        return out


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description="Feed given token ids through a model step by step and write logits.")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each rounded up to a multiple of 64")
    ap.add_argument("--page-size", type=int, default=16)
    args = ap.parse_args(argv)
    replayer = TraceReplayer(args.model, args.dtype, args.max_tokens, page_size=args.page_size)
    return replay_lines(replayer, sys.stdin, args.out)


def replay_lines(replayer: TraceReplayer, lines, out_dir: str) -> int:
    """Steps as JSON objects, one a line; `<step>.f32` into `out_dir` for every step that wants rows, and a line
    `done <step>` on standard output after every step."""
    os.makedirs(out_dir, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        logits = replayer.step(record)
        if logits is not None and logits.shape[0] > 0:
            logits.tofile(os.path.join(out_dir, f"{record['step']}.f32"))
        elif torch.cuda.is_available():
            torch.cuda.synchronize()
        print(f"done {record['step']}", flush=True)
    return 0
