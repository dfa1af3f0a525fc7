"""Shared by the CPU (emulated kernels) and GPU replay tests: run traces through
a TraceReplayer and compare every wanted row with the plain implementation."""
from __future__ import annotations

import torch

from plain_llama import plain_forward, read_model_folder
from replay_cases import collect, live_token_need

# How far logits may be from the plain implementation (float64), relative to the
# largest logit of the sequence.  float32: rounding of 32-bit sums only.
# bfloat16: activations are rounded to 8 bits of mantissa between kernels; the
# emulated kernels, which round at the same places, measure 0.25-0.45 %.
TOLERANCE = {"float32": 3e-5, "bfloat16": 1.5e-2}


def reference_rows(folder, requests):
    cfg, weights = read_model_folder(folder)
    return {rid: plain_forward(cfg, weights, toks) for rid, toks in requests.items()}


def run_trace(make_replayer, steps, max_tokens=None):
    replayer = make_replayer(max_tokens if max_tokens is not None else live_token_need(steps))
    outputs = []
    for step in steps:
        out = replayer.step(step)
        outputs.append(None if out is None else torch.from_numpy(out.copy()))
    return collect(steps, outputs), replayer


def check_rows(rows, reference, dtype, requests):
    worst = 0.0
    for rid, toks in requests.items():
        ref = reference[rid]
        scale = max(float(ref.abs().max()), 1.0)
        assert sorted(rows[rid]) == list(range(len(toks))), f"request {rid}: positions {sorted(rows[rid])[:5]}.. are not all of 0..{len(toks) - 1}"
        got = torch.stack([rows[rid][p] for p in range(len(toks))]).double()
        err = (got - ref).abs().max(dim=1).values / scale
        bad = (err > TOLERANCE[dtype]).nonzero()
        assert len(bad) == 0, (f"request {rid}: first wrong position {int(bad[0])} of {len(toks)} "
                               f"(error {float(err[int(bad[0])]):.3e} of the largest logit, allowed {TOLERANCE[dtype]:.1e}); "
                               f"{len(bad)} positions wrong")
        worst = max(worst, float(err.max()))
    return worst
