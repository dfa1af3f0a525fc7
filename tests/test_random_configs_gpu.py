"""Random configurations through the engine against the plain implementation: head sizes in steps of 16 from 16 to 256,
odd numbers of heads and of heads to a kv head, widths, intermediates and vocabularies that are no power of two (some
no multiple of 32 or 64, which sends products to other kernels), one to three layers, three rotation bases, with and
without llama3 scaling, tied and untied, three values of eps; each stepped by a random schedule (single tokens, short
and long portions mixed, up to four live requests on so few pages that they are used again) in float32 and bfloat16.
The two tiny configurations of the other tests differ in every option; these ask what happens in between."""
import random

import pytest
import torch

from llm_rs_amd import Engine, LlamaConfig
from plain_llama import plain_forward
from replay_checks import logit_scale, note, tolerance_for
from test_random_traces_gpu import random_schedule

pytestmark = pytest.mark.gpu
MAX_LIVE = 4


def random_config(seed: int) -> dict:
    rnd = random.Random(seed)
    kv = rnd.choice([1, 2, 3, 5, 8])
    d = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=rnd.randint(1, 3), hidden_size=8 * rnd.randint(4, 96),
             num_attention_heads=kv * rnd.choice([1, 2, 3, 4, 5, 7, 8]), num_key_value_heads=kv,
             head_dim=rnd.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256]), intermediate_size=8 * rnd.randint(4, 200),
             vocab_size=rnd.randint(300, 3000), rope_theta=rnd.choice([10000.0, 500000.0, 1234.5]), max_position_embeddings=2048,
             rms_norm_eps=rnd.choice([1e-5, 1e-6, 3e-4]), tie_word_embeddings=rnd.random() < 0.5)
    if rnd.random() < 0.5:
        d["rope_scaling"] = dict(rope_type="llama3", factor=rnd.choice([8.0, 32.0]), low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=rnd.choice([64, 256, 1024]))
    return d


@pytest.mark.parametrize("seed", [1, 2, 3, 5, 8, 13, 21, 34, 55, 89, 144, 233, 377, 610, 987, 4, 6, 7, 9, 10, 11, 12, 14, 15])
def test_a_random_configuration(seed):
    d = random_config(seed)
    cfg = LlamaConfig.from_dict(d)
    rnd = random.Random(seed + 1000)
    lens = [rnd.choice([1, 2, 16, 17, 64, 65, 129, 300])] + [rnd.randint(3, 260) for _ in range(5)]
    g = torch.Generator().manual_seed(seed)
    seqs = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lens]
    pages = sum(sorted(-(-n // 16) + 1 for n in lens)[-MAX_LIVE:]) + 1
    rows, weights = {}, None
    import test_random_traces_gpu
    was, test_random_traces_gpu.MAX_LIVE = test_random_traces_gpu.MAX_LIVE, MAX_LIVE
    try:
        for dtype in ("float32", "bfloat16"):
            eng = Engine.from_random(cfg, 7, dtype=dtype, page_size=16, num_pages=pages, max_requests=MAX_LIVE + 1, max_batch_tokens=4096)
            if weights is None:
                weights = {n: t.double() for n, t in eng.weights().items()}
            rows[dtype] = random_schedule(eng, seqs, seed * 7 + 1)
            core = eng.cache.core
            assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
            del eng
    finally:
        test_random_traces_gpu.MAX_LIVE = was
    reference = [plain_forward(d, weights, s) for s in seqs]
    stored = {n: t.bfloat16() if t.dim() > 1 else t.float() for n, t in weights.items()}
    for dtype in ("float32", "bfloat16"):
        allowed = tolerance_for(dtype, d, stored, seqs[:3])
        for (r, p), row in rows[dtype].items():
            err = float((row.double() - reference[r][p]).abs().max()) / logit_scale(reference[r])
            note(dtype, err)
            assert err <= allowed, (f"{dtype}, configuration {d}: request {r} (length {lens[r]}) position {p}: {err:.3e} of the "
                                    f"largest logit, allowed {allowed:.3e}")
