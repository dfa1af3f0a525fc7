"""Random traces at widths where the kernels for wide layers run: requests of random lengths, stepped in random
batches (a random subset of up to ten live requests each step; single tokens, short portions and long ones mixed by
a random rule), few pages so that they are used again, against the plain implementation on every wanted row.
The fixed cuts of the replay tests meet each kernel at a handful of batch sizes; these meet them at whatever comes."""
import random

import pytest
import torch

from llm_rs_amd import Engine, LlamaConfig, StepEntry
from plain_llama import plain_forward
from replay_checks import logit_scale, note, tolerance_for

pytestmark = pytest.mark.gpu
MAX_LIVE = 10


def random_schedule(eng, seqs, seed):
    """Steps `seqs` through the engine to their ends; returns {(request, position): logits row}."""
    rnd = random.Random(seed)
    lens = [len(s) for s in seqs]
    waiting, live, got = list(range(len(seqs))), {}, {}
    while waiting or live:
        while waiting and len(live) < MAX_LIVE and (not live or rnd.random() < 0.5):
            live[waiting.pop(0)] = [eng.open_request(), 0]
        chosen = [r for r in live if rnd.random() < 0.8] or [next(iter(live))]
        mode = rnd.random()
        entries, meta = [], []
        for r in chosen:
            slot, pos = live[r]
            left = lens[r] - pos
            if mode < 0.45:
                n = 1
            elif mode < 0.75:
                n = 1 if rnd.random() < 0.7 else rnd.randint(2, 40)
            else:
                n = rnd.choice([1, 1, 2, 3, 17, 33, 64, 100, 200, 256, 300])
            n = min(n, left)
            want = sorted({n - 1, rnd.randrange(n)})
            entries.append(StepEntry(slot, pos, seqs[r][pos:pos + n], want))
            meta.append((r, pos, n, want))
        out = eng.step(entries).float().cpu()
        row = 0
        for r, pos, n, want in meta:
            for w in want:
                got[(r, pos + w)] = out[row].clone()
                row += 1
            live[r][1] += n
            if live[r][1] >= lens[r]:
                eng.close_request(live[r][0])
                del live[r]
    return got


@pytest.mark.parametrize("hidden,inter,heads,kv,hd,layers,seed", [(2048, 4096, 16, 4, 128, 2, 3), (1024, 2816, 8, 2, 128, 3, 9),
                                                                 (2048, 8192, 32, 8, 64, 1, 7)])
def test_random_traces(hidden, inter, heads, kv, hd, layers, seed):
    cfg = LlamaConfig.from_dict(dict(
        architectures=["LlamaForCausalLM"], num_hidden_layers=layers, hidden_size=hidden, num_attention_heads=heads,
        num_key_value_heads=kv, head_dim=hd, intermediate_size=inter, vocab_size=640, rope_theta=500000.0,
        max_position_embeddings=4096, rms_norm_eps=1e-5, tie_word_embeddings=False))
    rnd = random.Random(seed)
    lens = [1300, 64] + [rnd.randint(40, 700) for _ in range(20)]
    g = torch.Generator().manual_seed(seed)
    seqs = [torch.randint(0, 640, (n,), generator=g).tolist() for n in lens]
    pages = sum(sorted(-(-n // 16) + 1 for n in lens)[-MAX_LIVE:]) + 2          # what the ten longest need: the rest reuse
    rows, weights = {}, None
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_random(cfg, 7, dtype=dtype, page_size=16, num_pages=pages, max_requests=MAX_LIVE + 2, max_batch_tokens=4096)
        if weights is None:
            weights = {n: t.double() for n, t in eng.weights().items()}
        rows[dtype] = random_schedule(eng, seqs, seed * 7 + 1)
        del eng
    reference = [plain_forward(cfg.to_dict(), weights, s) for s in seqs]
    for dtype in ("float32", "bfloat16"):
        allowed = tolerance_for(dtype, cfg.to_dict(), {n: t.bfloat16() if t.dim() > 1 else t.float() for n, t in weights.items()},
                                [seqs[1], seqs[2][:96]])
        for (r, p), row in rows[dtype].items():
            err = float((row.double() - reference[r][p]).abs().max()) / logit_scale(reference[r])
            note(dtype, err)
            assert err <= allowed, f"{dtype}: request {r} (length {lens[r]}) position {p}: {err:.3e} of the largest logit, allowed {allowed:.3e}"
