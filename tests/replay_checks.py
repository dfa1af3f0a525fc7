"""Shared by the CPU (emulated kernels) and GPU replay tests: run traces through
a TraceReplayer and compare every wanted row with the plain implementation."""
from __future__ import annotations

import torch

from plain_llama import plain_forward, read_model_folder
from replay_cases import collect, live_token_need

# How far logits may be from the plain implementation (float64), as a part of the
# largest logit of the sequence (the sequence's own scale, whatever it is: no floor).
# float32: rounding of 32-bit sums only, the same bound for every model.
# bfloat16: activations are rounded to 8 bits of mantissa between kernels, and how much of the
# largest logit that costs depends on the model (its width, its depth, how far its largest logit
# stands out).  So the bound is measured per model, not chosen: the emulated kernels
# (emulated_kernels.py: plain tensor operations on the host that round where the device's kernels
# round) run the same model on the same sequences, and the device may be BF16_FACTOR times as far
# from the plain implementation as they are: it sums in other orders and exponentiates in base 2,
# it does not round more often.
TOLERANCE = {"float32": 3e-5}
BF16_FACTOR = 2.0

# the worst error each dtype has shown in this run of the tests, for the summary at its end
WORST = {}


def logit_scale(ref) -> float:
    return float(ref.abs().max())


def note(dtype, err: float) -> None:
    WORST[dtype] = max(WORST.get(dtype, 0.0), float(err))


def emulated_bf16_error(cfg: dict, weights, sequences, reference=None) -> float:
    """The worst error of the emulated bfloat16 kernels on these whole sequences, as a part of each
    sequence's largest logit."""
    from emulated_kernels import EmulatedKernels
    from llm_rs_amd import Engine, StepEntry, config_from_dict, use_kernels
    longest = max(len(s) for s in sequences)
    worst = 0.0
    with use_kernels(EmulatedKernels()):
        eng = Engine(config_from_dict(cfg), weights, dtype="bfloat16", device="cpu", page_size=16,
                     num_pages=-(-longest // 16) + 1, max_requests=2)
        for i, seq in enumerate(sequences):
            ref = reference[i] if reference is not None else plain_forward(cfg, weights, seq)
            slot = eng.open_request()
            got = eng.step([StepEntry(slot, 0, list(seq), list(range(len(seq))))]).double()
            eng.close_request(slot)
            worst = max(worst, float((got - ref).abs().max()) / logit_scale(ref))
    return worst


def tolerance_for(dtype: str, cfg: dict, weights, sequences, reference=None) -> float:
    """The bound for a model-level comparison in `dtype` on this model and these sequences."""
    if dtype == "float32":
        return TOLERANCE["float32"]
    return BF16_FACTOR * emulated_bf16_error(cfg, weights, sequences, reference)


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
