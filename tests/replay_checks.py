"""Shared by the CPU (emulated kernels) and GPU replay tests: run traces through
a TraceReplayer and compare every wanted row with the plain implementation."""
from __future__ import annotations

import torch

from plain_llama import plain_forward, read_model_folder
from replay_cases import collect, live_token_need

# How far logits may be from the plain implementation (float64), as a part of the
# largest logit of the sequence (the sequence's own scale, whatever it is: no floor).
# float32: rounding of 32-bit sums only: 3e-5 for every model, except that a deep one may need more room.  The
# error is round-off and grows with the square root of the depth: at the 8B shape's widths, 2 / 8 / 16 / 32 layers,
# the engine is 6.5e-6 / 1.5e-5 / 2.0e-5 / 2.7e-5 from the exact logits, and the plain implementation itself, run
# in float32, 5.9e-6 / 1.2e-5 / 1.9e-5 / 2.8e-5.  A test of a deep model therefore runs the plain implementation in
# float32 beside the exact pass (`also_in`) and allows F32_FACTOR times its distance where that is more than 3e-5.
# bfloat16: activations are rounded to 8 bits of mantissa between kernels, and how much of the
# largest logit that costs depends on the model (its width, its depth, how far its largest logit
# stands out).  So the bound is computed per model, and from nothing of the engine's: the plain
# implementation runs the same sequences a second time with every activation that passes from one
# kernel to the next rounded to bfloat16 (plain_llama.plain_forward_streamed, `rounding`), and the
# device may be BF16_FACTOR times as far from the exact result as that pass is: it sums in other
# orders and exponentiates in base 2, it does not round more often.
TOLERANCE = {"float32": 3e-5}
BF16_FACTOR = 1.5
F32_FACTOR = 1.5

# the worst error each dtype has shown in this run of the tests, for the summary at its end
WORST = {}


def logit_scale(ref) -> float:
    return float(ref.abs().max())


def note(dtype, err: float) -> None:
    WORST[dtype] = max(WORST.get(dtype, 0.0), float(err))


def rounding_error(cfg: dict, weights, sequences, rounding=torch.bfloat16, device="cpu") -> float:
    """How far rounding of the activations to `rounding` alone takes this model on these whole sequences from the
    exact result, as a part of each sequence's largest logit (the worst of them)."""
    from plain_llama import plain_forward_streamed
    exact, rounded = plain_forward_streamed(cfg, lambda name: weights[name], sequences, rounding=rounding, device=device)
    return max(float((a - b).abs().max()) / logit_scale(a) for a, b in zip(exact, rounded))


def tolerance_for(dtype: str, cfg: dict, weights, sequences, reference=None) -> float:
    """The bound for a model-level comparison in `dtype` on this model and these sequences."""
    if dtype == "float32":
        return TOLERANCE["float32"]
    return BF16_FACTOR * rounding_error(cfg, weights, sequences)


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


def check_rows(rows, reference, dtype, requests, allowed=None):
    """`allowed`: the bound (see tolerance_for); without one, float32's."""
    allowed = TOLERANCE[dtype] if allowed is None else allowed
    worst = 0.0
    for rid, toks in requests.items():
        ref = reference[rid]
        scale = logit_scale(ref)
        assert sorted(rows[rid]) == list(range(len(toks))), f"request {rid}: positions {sorted(rows[rid])[:5]}.. are not all of 0..{len(toks) - 1}"
        got = torch.stack([rows[rid][p] for p in range(len(toks))]).double()
        err = (got - ref).abs().max(dim=1).values / scale
        bad = (err > allowed).nonzero()
        assert len(bad) == 0, (f"request {rid}: first wrong position {int(bad[0])} of {len(toks)} "
                               f"(error {float(err[int(bad[0])]):.3e} of the largest logit, allowed {allowed:.1e}); "
                               f"{len(bad)} positions wrong")
        worst = max(worst, float(err.max()))
    note(dtype, worst)
    if dtype == "bfloat16":
        note("bfloat16, of what is allowed", worst / allowed)
    return worst
