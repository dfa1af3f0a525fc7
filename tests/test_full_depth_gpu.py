"""The model that bench.py times, at its real depth: the Llama-3.1-8B shape with all 32 layers and the
full vocabulary, random weights, in float32 and bfloat16.

First the four ways of cutting (whole; the last 32 tokens one by one; portions of changing size; mixed
with reused pages) on four short requests, every row compared with the plain implementation.  Then the
steps the benchmark runs, which no small model reaches: a prompt of 2,049 tokens and one of 1,025 in one
step each (whole rounds of the large tiles and one row more) and cut at 1,024, and a portion of 2,048
tokens beside sixteen requests that decode, as one step.

The engine makes its weights on the device from the seed; the plain implementation makes the same
tensors on the host, one layer at a time, from the same seed (the fill is the same function of seed and
index on both sides), and runs them in float64 with one layer in memory at a time: the same plain tensor
operations as everywhere, placed on the device for this file, where the 6,000 tokens of 32 layers take
seconds and not a quarter of an hour.  The same pass rounds a second set of activations to bfloat16
wherever one kernel hands them to the next; how far that alone takes these logits is what the bfloat16
bound is made from (replay_checks.BF16_FACTOR times it), and a third set is computed in float32 throughout:
what 32-bit sums alone cost at this depth, from which the float32 bound is made where it is more than the
3e-5 of every model (replay_checks.F32_FACTOR).  The file states no figure of its own."""
import time

import pytest
import torch

from llm_rs_amd import Engine, LlamaConfig, StepEntry
from llm_rs_amd.engine import Model
from llm_rs_amd.engine.trace import TraceReplayer
from llm_rs_amd.weights import random_tensors
from plain_llama import plain_forward_streamed
from replay_cases import live_token_need, mixed, portions, random_tokens, tail_decoded, whole
from replay_checks import BF16_FACTOR, F32_FACTOR, TOLERANCE, check_rows, logit_scale, note, run_trace

pytestmark = pytest.mark.gpu

LLAMA_8B = dict(
    architectures=["LlamaForCausalLM"], num_hidden_layers=32, hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=8192, rms_norm_eps=1e-5, tie_word_embeddings=False, hidden_act="silu")
LLAMA_1B = dict(LLAMA_8B, num_hidden_layers=16, hidden_size=2048, head_dim=64, intermediate_size=8192, tie_word_embeddings=True,
                rope_scaling=dict(LLAMA_8B["rope_scaling"], factor=32.0))
SEED = 0                       # bench.py's
LENGTHS = [33, 70, 100, 128]
LENGTHS_1B = [33, 70, 130, 300, 57]
N_DECODING = 16


def places(n):
    """The rows of a long request that are compared: the edges of every tile size, and a few between."""
    edges = [0, 1, 15, 16, 31, 32, 63, 64, 127, 128, 255, 256, 511, 512, 1023, 1024, 1025, 2047, 2048]
    return sorted({p for p in edges + list(range(97, n, 193)) + [n - 2, n - 1] if 0 <= p < n})


def make_case(config: dict, lengths, with_long: bool):
    cfg = LlamaConfig.from_dict(config)
    V = cfg.vocab_size
    requests = {f"r{i}": random_tokens(V, n, seed=80 + i) for i, n in enumerate(lengths)}
    long = {}
    if with_long:
        long = {"a": random_tokens(V, 2049, seed=90), "b": random_tokens(V, 1025, seed=91), "c": random_tokens(V, 2048, seed=92)}
        long.update({f"d{i}": random_tokens(V, 40 + i, seed=100 + i) for i in range(N_DECODING)})
    specs = Model(cfg.model_spec(), torch.bfloat16, "cpu").tensors()
    t0 = time.time()

    def host_tensor(name):      # the tensor random-weights mode gives `name`, made here, on the host
        return random_tensors({name: specs[name].shape}, {name: specs[name].kind}, SEED, device="cpu")[name]

    names = list(requests) + list(long)
    wanted = [list(range(len(requests[r]))) for r in requests] + [places(len(long[r])) for r in long]
    exact, rounded, in32 = plain_forward_streamed(cfg.to_dict(), host_tensor, [{**requests, **long}[r] for r in names], rows=wanted,
                                                  rounding=torch.bfloat16, device="cuda", also_in=torch.float32)
    reference = {r: e.cpu() for r, e in zip(names, exact)}
    by_rounding = {r: (float((e - y).abs().max()) / logit_scale(e), float((e - z.double()).abs().max()) / logit_scale(e))
                   for r, e, y, z in zip(names, exact, rounded, in32)}
    del exact, rounded, in32
    torch.cuda.empty_cache()
    print(f"plain implementation, {cfg.num_hidden_layers} layers, {sum(len(w) for w in wanted)} rows of {sum(len({**requests, **long}[r]) for r in names)} tokens: "
          f"{time.time() - t0:.0f}s; rounding to bfloat16 alone moves the logits by {max(b for b, _ in by_rounding.values()):.3e} of the largest, "
          f"computing in float32 by {max(f for _, f in by_rounding.values()):.3e}", flush=True)
    return cfg, requests, long, reference, by_rounding


@pytest.fixture(scope="module")
def case():
    return make_case(LLAMA_8B, LENGTHS, with_long=True)


def allowed_for(dtype, by_rounding, names):
    if dtype == "float32":
        return max(TOLERANCE["float32"], F32_FACTOR * max(by_rounding[r][1] for r in names))
    return BF16_FACTOR * max(by_rounding[r][0] for r in names)


def every_cut(cfg, requests, reference, by_rounding, dtype, num_pages):
    allowed = allowed_for(dtype, by_rounding, requests)
    engine = Engine.from_random(cfg, SEED, dtype=dtype, device="cuda", page_size=16, num_pages=num_pages, max_requests=8)
    assert len(engine.model.blocks) == cfg.num_hidden_layers and engine.model.head.shape == (cfg.vocab_size, cfg.hidden_size)
    cuts = {"whole": whole(requests), "tail": tail_decoded(requests, 32), "portions": portions(requests),
            "mixed": mixed(requests, live=4)}
    total = sum(-(-len(t) // 64) * 64 for t in requests.values())
    for name, steps in cuts.items():
        need = live_token_need(steps)
        assert need <= num_pages * 16
        if name == "mixed":
            assert need < total + 64, "so few pages that they are used again"
        # the same engine for every cut: what a cut leaves in the pages must not show in the next
        rows, rep = run_trace(lambda n: TraceReplayer.for_engine(engine), steps)
        worst = check_rows(rows, reference, dtype, requests, allowed)
        print(f"{dtype} {name}: worst error {worst:.3e} of the largest logit (allowed {allowed:.1e})", flush=True)
        core = engine.cache.core
        assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
    return engine


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_benchmarked_model_in_every_cut(case, dtype):
    cfg, requests, _, reference, by_rounding = case
    every_cut(cfg, requests, reference, by_rounding, dtype, num_pages=64)


@pytest.fixture(scope="module")
def case_1b():
    return make_case(LLAMA_1B, LENGTHS_1B, with_long=False)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_1b_shape_at_full_depth_in_every_cut(case_1b, dtype):
    """The serving benchmark's model as it is: 16 layers, head size 64, the output matrix tied to the token table of
    128,256 rows, frequencies scaled by 32."""
    cfg, requests, _, reference, by_rounding = case_1b
    engine = every_cut(cfg, requests, reference, by_rounding, dtype, num_pages=48)
    assert engine.model.head is engine.model.embedding


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_steps_the_benchmark_runs(case, dtype):
    """Steps of 2,049, 1,025 and 2,048 + 16 rows through all 32 layers: the large tiles with their rows beyond whole
    tiles handed to the few-row kernel, the prompt attention over 128 pages, the rotation kernel of many rows, the
    second stream for the decoding requests' attention, workspaces grown to such steps."""
    cfg, _, long, reference, by_rounding = case
    allowed = allowed_for(dtype, by_rounding, long)
    engine = Engine.from_random(cfg, SEED, dtype=dtype, device="cuda", page_size=16, num_pages=360, max_requests=32)
    core = engine.cache.core
    worst = {}

    def compare(name, rid, got, at):
        """`got`: logits of the rows `at` (places of request `rid`, a subset of those the reference holds)."""
        ref_rows = places(len(long[rid]))
        ref = reference[rid][[ref_rows.index(p) for p in at]]
        err = (got.double().cpu() - ref).abs().max(dim=1).values / logit_scale(reference[rid])
        bad = (err > allowed).nonzero()
        assert len(bad) == 0, (f"{dtype}, {name}, request {rid}: first wrong position {at[int(bad[0])]} (error {float(err[int(bad[0])]):.3e} "
                               f"of the largest logit, allowed {allowed:.1e}); {len(bad)} of {len(at)} rows wrong")
        worst[name] = max(worst.get(name, 0.0), float(err.max()))

    def run_cut(name, rid, cuts):
        slot, pos = engine.open_request(), 0
        for n in cuts:
            at = [p for p in places(len(long[rid])) if pos <= p < pos + n]
            got = engine.step([StepEntry(slot, pos, long[rid][pos:pos + n], [p - pos for p in at])])
            compare(name, rid, got, at)
            pos += n
        engine.close_request(slot)

    run_cut("2049 whole", "a", [2049])
    run_cut("2049 as 1024 + 1025", "a", [1024, 1025])
    run_cut("1025 whole", "b", [1025])
    run_cut("1025 as 1024 + 1", "b", [1024, 1])
    # sixteen requests up to their last token but one (as one step of sixteen portions), then one step:
    # a portion of 2,048 tokens and beside it each of the sixteen with its last token
    ds = [f"d{i}" for i in range(N_DECODING)]
    slots = {rid: engine.open_request() for rid in ds + ["c"]}
    got = engine.step([StepEntry(slots[rid], 0, long[rid][:-1], [len(long[rid]) - 2]) for rid in ds])
    for i, rid in enumerate(ds):
        compare("sixteen portions", rid, got[i:i + 1], [len(long[rid]) - 2])
    at_c = places(2048)
    entries = [StepEntry(slots[rid], len(long[rid]) - 1, long[rid][-1:], [0]) for rid in ds[:8]]
    entries.append(StepEntry(slots["c"], 0, long["c"], at_c))
    entries += [StepEntry(slots[rid], len(long[rid]) - 1, long[rid][-1:], [0]) for rid in ds[8:]]
    got = engine.step(entries)
    assert got.shape[0] == len(at_c) + N_DECODING
    for i, rid in enumerate(ds[:8]):
        compare("2048 beside 16", rid, got[i:i + 1], [len(long[rid]) - 1])
    compare("2048 beside 16", "c", got[8:8 + len(at_c)], at_c)
    for i, rid in enumerate(ds[8:]):
        compare("2048 beside 16", rid, got[8 + len(at_c) + i:9 + len(at_c) + i], [len(long[rid]) - 1])
    for rid in slots:
        engine.close_request(slots[rid])
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
    for name, w in worst.items():
        print(f"{dtype} {name}: worst error {w:.3e} of the largest logit (allowed {allowed:.1e})", flush=True)
    note(dtype, max(worst.values()))
    if dtype == "bfloat16":
        note("bfloat16, of what is allowed", max(worst.values()) / allowed)
