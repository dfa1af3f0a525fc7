"""Decoding far into a context, through the engine: two layers of the 8B shape's widths, a prompt of 8,200 tokens
fed in portions of 2,048 (the later ones attend over thousands of keys that earlier steps left), then tokens one by
one past position 8,192, in float32 and bfloat16, against the plain implementation over the whole sequence.  Beyond
what the other model-level tests reach: block tables hundreds of pages wide, the decode attention's split over
many chunks and its merge, the prompt tiles at a large offset, llama3-scaled rotation at positions in the thousands."""
import pytest
import torch

from llm_rs_amd import Engine, LlamaConfig, StepEntry
from plain_llama import plain_forward_streamed
from replay_cases import random_tokens
from replay_checks import BF16_FACTOR, TOLERANCE, logit_scale, note

pytestmark = pytest.mark.gpu

CONFIG = dict(
    architectures=["LlamaForCausalLM"], num_hidden_layers=2, hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=3000, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=16384, rms_norm_eps=1e-5, tie_word_embeddings=False, hidden_act="silu")
PROMPT, DECODED, PORTION = 8200, 12, 2048


def test_decoding_past_8192_positions():
    cfg = LlamaConfig.from_dict(CONFIG)
    tokens = random_tokens(cfg.vocab_size, PROMPT + DECODED, seed=61)
    # rows compared: a few of every portion (its first, one inside, its last) and every decoded token
    wanted = sorted({p for lo in range(0, PROMPT, PORTION) for p in (lo, lo + 1000, min(lo + PORTION, PROMPT) - 1) if p < PROMPT}
                    | set(range(PROMPT, PROMPT + DECODED)))
    weights = reference = by_rounding = None
    for dtype in ("bfloat16", "float32"):
        engine = Engine.from_random(cfg, 21, dtype=dtype, page_size=16, num_pages=(PROMPT + DECODED) // 16 + 2, max_requests=4)
        if weights is None:
            weights = engine.weights()
            exact, rounded = plain_forward_streamed(cfg.to_dict(), lambda name: weights[name], [tokens], rows=[wanted],
                                                    rounding=torch.bfloat16, device="cuda")
            reference = exact[0].cpu()
            by_rounding = float((exact[0] - rounded[0]).abs().max()) / logit_scale(exact[0])
            del exact, rounded
            torch.cuda.empty_cache()
        allowed = TOLERANCE["float32"] if dtype == "float32" else BF16_FACTOR * by_rounding
        slot, got = engine.open_request(), {}
        for lo in range(0, PROMPT, PORTION):
            hi = min(lo + PORTION, PROMPT)
            at = [p for p in wanted if lo <= p < hi]
            out = engine.step([StepEntry(slot, lo, tokens[lo:hi], [p - lo for p in at])])
            got.update({p: out[i].double().cpu() for i, p in enumerate(at)})
        for p in range(PROMPT, PROMPT + DECODED):
            got[p] = engine.step([StepEntry(slot, p, [tokens[p]], [0])])[0].double().cpu()
        engine.close_request(slot)
        err = torch.stack([(got[p] - reference[i]).abs().max() for i, p in enumerate(wanted)]) / logit_scale(reference)
        bad = (err > allowed).nonzero()
        assert len(bad) == 0, (f"{dtype}: first wrong position {wanted[int(bad[0])]} (error {float(err[int(bad[0])]):.3e} of the largest "
                               f"logit, allowed {allowed:.1e}); {len(bad)} of {len(wanted)} rows wrong")
        print(f"{dtype}: worst error {float(err.max()):.3e} of the largest logit (allowed {allowed:.1e}), "
              f"decoded rows {float(err[-DECODED:].max()):.3e}", flush=True)
        note(dtype, float(err.max()))
        del engine
