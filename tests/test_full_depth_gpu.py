"""The model that bench.py times, at its real depth: the Llama-3.1-8B shape with all 32 layers and the
full vocabulary, random weights, in float32 and bfloat16, replayed in the four ways of cutting (whole;
the last 32 tokens one by one; portions of changing size; mixed with reused pages) and compared row by
row with the plain implementation.  The engine makes its weights on the device from the seed; the plain
implementation makes the same tensors on the host, one layer at a time, from the same seed (the fill is
the same function of seed and index on both sides), and runs in float64 with one layer in memory."""
import time

import pytest
import torch

from llm_rs_amd import Engine, LlamaConfig
from llm_rs_amd.engine import Model
from llm_rs_amd.engine.trace import TraceReplayer
from llm_rs_amd.weights import random_tensors
from plain_llama import plain_forward_streamed
from replay_cases import live_token_need, mixed, portions, random_tokens, tail_decoded, whole
from replay_checks import BF16_FACTOR, TOLERANCE, check_rows, run_trace

pytestmark = pytest.mark.gpu

LLAMA_8B = dict(
    architectures=["LlamaForCausalLM"], num_hidden_layers=32, hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=8192, rms_norm_eps=1e-5, tie_word_embeddings=False, hidden_act="silu")
SEED = 0                       # bench.py's
LENGTHS = [33, 70, 100, 128]
# float32: the bound of every model.  bfloat16: the small models get their bounds from the emulated kernels run
# beside the test; at this size that run takes minutes on the host, so its result is stated here instead: the
# emulated kernels are 4.63e-2 of the largest logit from the plain implementation on these four requests (random
# weights of this width and depth, logits of standard deviation 1.29 and a largest of 7: rounding to 8 bits
# between kernels costs that much), and the device may be BF16_FACTOR times as far, as everywhere.  (Measured
# on the device: 5.1e-2 whole, 4.6e-2 to 4.7e-2 in the other cuts.)
BF16_EMULATED = 4.63e-2
ALLOWED = {"float32": TOLERANCE["float32"], "bfloat16": BF16_FACTOR * BF16_EMULATED}


@pytest.fixture(scope="module")
def case():
    cfg = LlamaConfig.from_dict(LLAMA_8B)
    requests = {f"r{i}": random_tokens(cfg.vocab_size, n, seed=80 + i) for i, n in enumerate(LENGTHS)}
    specs = Model(cfg.model_spec(), torch.bfloat16, "cpu").tensors()
    t0 = time.time()

    def host_tensor(name):      # the tensor random-weights mode gives `name`, made here, on the host
        return random_tensors({name: specs[name].shape}, {name: specs[name].kind}, SEED, device="cpu")[name]

    rows = plain_forward_streamed(cfg.to_dict(), host_tensor, list(requests.values()))
    print(f"plain implementation, 32 layers, {sum(LENGTHS)} tokens: {time.time() - t0:.0f}s", flush=True)
    return cfg, requests, dict(zip(requests, rows))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_benchmarked_model_in_every_cut(case, dtype):
    cfg, requests, reference = case
    engine = Engine.from_random(cfg, SEED, dtype=dtype, device="cuda", page_size=16, num_pages=64, max_requests=8)
    assert engine.model.spec.schedule and len(engine.model.blocks) == 32 and engine.model.head.shape == (128256, 4096)
    cuts = {"whole": whole(requests), "tail": tail_decoded(requests, 32), "portions": portions(requests),
            "mixed": mixed(requests, live=4)}
    total = sum(-(-n // 64) * 64 for n in LENGTHS)
    for name, steps in cuts.items():
        need = live_token_need(steps)
        assert need <= 64 * 16
        if name == "mixed":
            assert need < total + 64, "so few pages that they are used again"
        # the same engine for every cut: what a cut leaves in the pages must not show in the next
        rows, rep = run_trace(lambda n: TraceReplayer.for_engine(engine), steps)
        worst = check_rows(rows, reference, dtype, requests, ALLOWED[dtype])
        print(f"{dtype} {name}: worst error {worst:.3e} of the largest logit (allowed {ALLOWED[dtype]:.1e})", flush=True)
        core = engine.cache.core
        assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
