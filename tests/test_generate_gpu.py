"""Generation through the Python entry point: greedy against the plain
implementation, long decoding, the first tokens of a sequence, batching that
does not change outputs, seeds that reproduce, a pool so small that requests are
preempted and computed again."""
import pytest
import torch

from llm_rs_amd import Engine, StepEntry
from plain_llama import plain_forward, plain_generate, read_model_folder
from replay_cases import random_tokens
from replay_checks import TOLERANCE, logit_scale, note, tolerance_for
from tiny_configs import CONFIGS, PAGE_SIZE, make_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    d = tmp_path_factory.mktemp("models")
    return {w: make_folder(d, w, seed=7) for w in "AB"}


def engine(folder, which, dtype, **kw):
    kw.setdefault("num_pages", 256)
    kw.setdefault("max_requests", 16)
    return Engine.from_folder(folder, dtype=dtype, page_size=PAGE_SIZE[which], **kw)


def check_greedy_path(cfg, weights, prompt, out, dtype):
    """Every generated token is the plain implementation's choice given the same
    prefix, or (bfloat16) so close to it that rounding decides."""
    logits = plain_forward(cfg, weights, prompt + out)
    scale = logit_scale(logits)
    allowed = tolerance_for(dtype, cfg, weights, [prompt + out], [logits])
    for i, tok in enumerate(out):
        row = logits[len(prompt) - 1 + i]
        gap = float(row.max() - row[tok])
        assert gap <= allowed * scale, f"token {i}: engine chose {tok}, plain prefers {int(row.argmax())} by {gap}"


@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_matches_plain_float32(folders, which):
    cfg, weights = read_model_folder(folders[which])
    eng = engine(folders[which], which, "float32")
    lengths = {"A": [5, 17, 33], "B": [1, 7, 64]}[which]
    prompts = [random_tokens(cfg["vocab_size"], n, seed=n) for n in lengths]
    got = eng.generate(prompts, max_new_tokens=16)
    for p, out in zip(prompts, got):
        assert len(out) == 16
        check_greedy_path(cfg, weights, p, out, "float32")
    want = [plain_generate(cfg, weights, p, 16) for p in prompts[:2]]
    assert got[:2] == want


@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_bfloat16(folders, which):
    cfg, weights = read_model_folder(folders[which])
    eng = engine(folders[which], which, "bfloat16")
    prompts = [random_tokens(cfg["vocab_size"], n, seed=100 + n) for n in (3, 20, 41)]
    for p, out in zip(prompts, eng.generate(prompts, max_new_tokens=24)):
        check_greedy_path(cfg, weights, p, out, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """A short prompt and then hundreds of tokens one by one, to the model's last position."""
    which = "B"
    cfg, weights = read_model_folder(folders[which])
    toks = random_tokens(cfg["vocab_size"], cfg["max_position_embeddings"], seed=1)
    ref = plain_forward(cfg, weights, toks)
    eng = engine(folders[which], which, dtype)
    s = eng.open_request()
    rows = [eng.step([StepEntry(s, 0, toks[:9], list(range(9)))]).clone()]
    for i in range(9, len(toks)):
        rows.append(eng.step([StepEntry(s, i, [toks[i]], [0])]).clone())
    eng.close_request(s)
    got = torch.cat(rows).double().cpu()
    err = (got - ref).abs().max(dim=1).values / logit_scale(ref)
    bad = (err > tolerance_for(dtype, cfg, weights, [toks], [ref])).nonzero()
    assert len(bad) == 0, f"first wrong position {int(bad[0])}: {float(err[int(bad[0])])}"
    note(dtype, err.max())
    with pytest.raises(ValueError, match="beyond the model"):
        s = eng.open_request()
        eng.step([StepEntry(s, 0, toks + [1], [])])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens(folders, dtype):
    """Positions 0, 1, 2: one-token prompts, alone and side by side."""
    which = "A"
    cfg, weights = read_model_folder(folders[which])
    eng = engine(folders[which], which, dtype)
    seqs = [random_tokens(cfg["vocab_size"], 3, seed=s) for s in range(4)]
    slots = [eng.open_request() for _ in seqs]
    scale_tol = tolerance_for(dtype, cfg, weights, seqs)
    for pos in range(3):
        out = eng.step([StepEntry(s, pos, [seq[pos]], [0]) for s, seq in zip(slots, seqs)]).double().cpu()
        for i, seq in enumerate(seqs):
            ref = plain_forward(cfg, weights, seq[:pos + 1])[-1]
            assert float((out[i] - ref).abs().max()) <= scale_tol * logit_scale(ref), (pos, i)


def test_batching_and_seeds_do_not_change_outputs(folders):
    which = "B"
    cfg, _ = read_model_folder(folders[which])
    prompts = [random_tokens(cfg["vocab_size"], n, seed=50 + n) for n in (1, 7, 64, 130, 300)]
    kw = dict(max_new_tokens=24, temperature=0.8, top_k=40, top_p=0.9, seed=42)
    together = engine(folders[which], which, "float32", max_chunk=32).generate(prompts, **kw)
    alone_eng = engine(folders[which], which, "float32")
    alone = [alone_eng.generate([p], **kw)[0] for p in prompts]
    assert together == alone, "a request's tokens do not depend on what it is batched with or how its prompt was cut"
    assert together == engine(folders[which], which, "float32", max_chunk=32).generate(prompts, **kw), "same seed, same tokens"
    other = alone_eng.generate(prompts, **{**kw, "seed": 43})
    assert other != together, "another seed draws other tokens"
    per_request = alone_eng.generate(prompts[:2], **{**kw, "seed": [42, 43]})
    assert per_request[0] == together[0] and per_request[1] == other[1]
    limits = [5, 0, 24, 1, 13]                                   # a limit for each request
    cut = alone_eng.generate(prompts, **{**kw, "max_new_tokens": limits})
    assert cut == [t[:m] for t, m in zip(together, limits)]


def test_sampled_tokens_follow_the_plain_sampler(folders):
    """Temperature sampling end to end in float32: the same tokens as the plain
    implementation drawing from the same generator."""
    which = "A"
    cfg, weights = read_model_folder(folders[which])
    eng = engine(folders[which], which, "float32")
    prompt = random_tokens(cfg["vocab_size"], 6, seed=3)
    got = eng.generate([prompt], max_new_tokens=12, temperature=0.8, seed=7)[0]
    assert got == plain_generate(cfg, weights, prompt, 12, temperature=0.8, seed=7)
    got = eng.generate([prompt], max_new_tokens=12, temperature=1.1, top_k=5, top_p=0.7, seed=0)[0]
    assert got == plain_generate(cfg, weights, prompt, 12, temperature=1.1, top_k=5, top_p=0.7, seed=0)


def test_stop_tokens_and_reasons(folders):
    which = "B"
    cfg, weights = read_model_folder(folders[which])
    eng = engine(folders[which], which, "float32")
    prompt = random_tokens(cfg["vocab_size"], 7, seed=9)
    free = eng.generate([prompt], max_new_tokens=10)[0]
    res = eng.generate([prompt], max_new_tokens=10, stop_token_ids=[free[4]], return_reasons=True)[0]
    first = free.index(free[4])
    assert res.tokens == free[:first] and res.reason == "stop", "the stop token ends the output and is not part of it"
    assert eng.generate([prompt], max_new_tokens=3, return_reasons=True)[0].reason == "length"
    assert eng.generate([prompt], max_new_tokens=0) == [[]]


def test_small_pool_preempts_and_recomputes(folders):
    """So few pages that running requests cannot all grow: some are evicted, wait, and are
    computed again; every output equals the run with plenty of pages."""
    which = "B"
    cfg, _ = read_model_folder(folders[which])
    prompts = [random_tokens(cfg["vocab_size"], n, seed=70 + n) for n in (30, 45, 20, 60, 10, 33)]
    kw = dict(max_new_tokens=40, temperature=0.7, seed=5)
    roomy = engine(folders[which], which, "float32").generate(prompts, **kw)
    tight = engine(folders[which], which, "float32", num_pages=14, max_chunk=16)      # 224 token slots for ~480 tokens of need
    assert tight.generate(prompts, **kw) == roomy
    assert tight.last_stats.preemptions > 0, "the case must make the scheduler evict"
    core = tight.cache.core
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
    with pytest.raises(Exception, match="pages"):
        tight.generate([random_tokens(cfg["vocab_size"], 200, seed=1)], max_new_tokens=100)


@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("B", "bfloat16"), ("B", "float32")])
def test_steps_started_ahead_change_no_output(folders, which, dtype):
    """A step planned and started while the step before it is in flight (its samples handed over on the device, the
    default) against stepping in turn: the same tokens and reasons, greedy and with a temperature, with a stop token
    that ends a request in the middle, recorded decode steps included, and with a pool so small that requests give way."""
    cfg, _ = read_model_folder(folders[which])
    prompts = [random_tokens(cfg["vocab_size"], n, seed=40 + n) for n in (5, 61, 18, 1, 33, 90, 7, 24)]
    limits = [40, 12, 1, 35, 20, 2, 30, 16]
    seeds = list(range(11, 19))

    def run(overlap, temperature, stop, **kw):
        eng = engine(folders[which], which, dtype, overlap=overlap, max_batch_tokens=64, **kw)
        got = eng.generate(prompts, limits, temperature=temperature, top_k=50, top_p=0.95, seed=seeds, stop_token_ids=stop,
                           return_reasons=True)
        core = eng.cache.core
        assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0 and not core.in_flight()
        return [(f.tokens, f.reason) for f in got], eng

    for temperature in (0.0, 0.8):
        free, _ = run(False, temperature, [])
        ahead, eng = run(True, temperature, [])
        assert ahead == free
        assert eng.runner.graph_replays > 0, "the case itself: decode steps that were recorded"
        found = [(i, j) for i, (toks, _) in enumerate(free) for j in range(1, len(toks)) if toks[j] not in toks[:j]]
        if found:
            i, at = found[0]
            stop = [free[i][0][at]]
            in_turn, _ = run(False, temperature, stop)
            assert in_turn[i] == (free[i][0][:at], "stop")
            assert run(True, temperature, stop)[0] == in_turn
        else:
            assert temperature == 0.0, "sampled outputs do bring new tokens"
    if dtype != "float32":
        return      # (in bfloat16 a request computed again after giving way meets other roundings, and when it gives way differs)
    tight_kw = dict(num_pages=12 if PAGE_SIZE[which] >= 16 else 12 * 16 // PAGE_SIZE[which], max_chunk=16)
    in_turn, eng = run(False, 0.8, [], **tight_kw)
    assert eng.last_stats.preemptions > 0, "the case itself: requests give way"
    assert run(True, 0.8, [], **tight_kw)[0] == in_turn


def test_a_dead_row_beside_sixteen_live_ones_moves_logits_by_rounding_only():
    """A step started ahead carries a row for a request that a stop token has just ended, so sixteen live requests
    run as a step of seventeen rows where stepping in turn runs sixteen; and the kernels choose by the row count (up to
    sixteen rows the norms are finished by the neighbouring products, from seventeen on by a norm kernel or by the
    product that is split over blocks).  The live rows' logits may differ between the two by rounding, not more:
    both are compared with the plain implementation and with each other, in bfloat16 and in float32."""
    from llm_rs_amd import LlamaConfig
    cfg = LlamaConfig.from_dict(dict(
        architectures=["LlamaForCausalLM"], num_hidden_layers=2, hidden_size=2048, num_attention_heads=16,
        num_key_value_heads=4, head_dim=128, intermediate_size=4096, vocab_size=1000, rope_theta=500000.0,
        max_position_embeddings=512, rms_norm_eps=1e-5, tie_word_embeddings=False))
    plen, n_live = 40, 16
    prompts = [random_tokens(1000, plen + 1, seed=500 + i) for i in range(n_live + 1)]
    weights = None
    for dtype in ("bfloat16", "float32"):
        eng = Engine.from_random(cfg, 9, dtype=dtype, page_size=16, num_pages=128, max_requests=32)
        if weights is None:
            weights = eng.weights()
        slots = [eng.open_request() for _ in prompts]
        for s, p in zip(slots, prompts):
            eng.step([StepEntry(s, 0, p[:plen], [])])
        decode = lambda n: [StepEntry(slots[i], plen, [prompts[i][plen]], [0]) for i in range(n)]
        in_turn = eng.step(decode(n_live)).double().cpu().clone()
        # the dead row stands in the middle, as a request that ended does, not at the end
        order = list(range(8)) + [n_live] + list(range(8, n_live))
        with_dead = eng.step([decode(n_live + 1)[i] for i in order]).double().cpu().clone()
        with_dead = with_dead[[order.index(i) for i in range(n_live)]]
        plain = torch.stack([plain_forward(cfg.to_dict(), {n: t.double() for n, t in weights.items()}, p)[-1] for p in prompts[:n_live]])
        allowed = tolerance_for(dtype, cfg.to_dict(), weights, prompts[:3])
        scale = logit_scale(plain)
        for name, a, b in (("in turn", in_turn, plain), ("with a dead row", with_dead, plain), ("one against the other", in_turn, with_dead)):
            err = float((a - b).abs().max()) / scale
            assert err <= allowed, f"{dtype}, {name}: {err:.3e} of the largest logit, allowed {allowed:.3e}"
            note(dtype, err)


@pytest.mark.parametrize("which,dtype", [("B", "bfloat16"), ("A", "float32")])
def test_recorded_decode_steps_equal_eager_ones(folders, which, dtype):
    """Decode steps are recorded into a HIP graph and replayed.  Every replay is compared
    with the same step run eagerly by a second engine, with eager prompt steps, new
    requests and synchronisations between the replays."""
    cfg, _ = read_model_folder(folders[which])
    recorded, eager = engine(folders[which], which, dtype), engine(folders[which], which, dtype)
    eager.runner.use_graphs = False
    assert recorded.runner.use_graphs
    seqs = [random_tokens(cfg["vocab_size"], 90, seed=200 + i) for i in range(3)]

    def both(make_entries):
        a = recorded.step(make_entries(slots_r)).clone()
        b = eager.step(make_entries(slots_e)).clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b)

    slots_r = [recorded.open_request() for _ in seqs]
    slots_e = [eager.open_request() for _ in seqs]
    both(lambda sl: [StepEntry(sl[i], 0, seqs[i][:20 + i], [19 + i]) for i in range(3)])
    pos = [20, 21, 22]
    for step in range(40):
        both(lambda sl: [StepEntry(sl[i], pos[i], [seqs[i][pos[i]]], [0]) for i in range(3)])
        pos = [p + 1 for p in pos]
        if step == 15:       # a prompt portion for one request between the replays: an eager step in both engines
            both(lambda sl: [StepEntry(sl[0], pos[0], seqs[0][pos[0]:pos[0] + 9], [8])])
            pos[0] += 9
        if step == 25:       # another batch size: another graph
            both(lambda sl: [StepEntry(sl[i], pos[i], [seqs[i][pos[i]]], [0]) for i in range(2)])
            pos[0] += 1; pos[1] += 1
    assert recorded.runner.graph_replays >= 30 and eager.runner.graph_replays == 0


def test_a_recording_is_kept_for_the_chunk_it_was_made_with():
    """The kernel library shares a decoding request's keys out over waves in chunks whose length it chooses by how
    many keys the step sees, and a recorded step holds the chunk it was recorded with.  Sixteen requests decode from
    twenty keys before the length where that choice changes: the runner records a second graph for the same sizes
    there, and every step's logits stay those of an engine that records nothing."""
    from llm_rs_amd import LlamaConfig
    from llm_rs_amd.kernels import kernels
    cfg = LlamaConfig.from_dict(dict(
        architectures=["LlamaForCausalLM"], num_hidden_layers=1, hidden_size=512, num_attention_heads=8,
        num_key_value_heads=8, head_dim=64, intermediate_size=512, vocab_size=500, rope_theta=10000.0,
        max_position_embeddings=4096, rms_norm_eps=1e-5, tie_word_embeddings=True))
    n_req, steps = 16, 40
    k = kernels()
    by_len = [k.attention_split_chunk(n_req, 8, 64, 2048, n_req * n) for n in range(300, 1990)]
    change = next(300 + i + 1 for i, (a, b) in enumerate(zip(by_len, by_len[1:])) if a != b)
    plen = change - 20           # (with the rule as it stands: 902)
    chunks = {k.attention_split_chunk(n_req, 8, 64, 2048, n_req * (plen + 1 + i)) for i in range(steps)}
    assert len(chunks) == 2, "the case itself: the chunk must change on the way"
    prompts = [random_tokens(500, plen + steps + 1, seed=900 + i) for i in range(n_req)]
    recorded = Engine.from_random(cfg, 11, dtype="bfloat16", page_size=16, num_pages=n_req * 128 + 8, max_requests=16)
    eager = Engine.from_random(cfg, 11, dtype="bfloat16", page_size=16, num_pages=n_req * 128 + 8, max_requests=16)
    eager.runner.use_graphs = False
    for block in recorded.model.blocks:          # (a batch would keep its first chunk for 256 steps otherwise)
        block.mixer.chunk_patience = 3
    slots = {}
    for eng in (recorded, eager):
        slots[eng] = [eng.open_request() for _ in range(n_req)]
        for s, p in zip(slots[eng], prompts):
            eng.step([StepEntry(s, 0, p[:plen], [])])
    seen = set()
    for i in range(steps):
        entries = lambda eng: [StepEntry(slots[eng][r], plen + i, [prompts[r][plen + i]], [0]) for r in range(n_req)]
        a = recorded.step(entries(recorded)).float().clone()
        b = eager.step(entries(eager)).float().clone()
        torch.cuda.synchronize()
        # (the eager engine bounds the lengths by the longest request, the recording one by its block-table width:
        # the chunks may differ, and with them the order of the sums)
        assert (a - b).abs().max() <= 2e-2 * b.abs().max(), f"step {i}"
        seen.add(len(recorded.runner._graphs))
    assert recorded.runner.graph_replays >= steps - 8
    assert max(seen) == 2, "one recording for each chunk"


@pytest.mark.parametrize("hidden,heads,inter,layers", [(4096, 32, 14336, 1), (8192, 64, 28672, 1), (2048, 32, 8192, 2)])
def test_layers_of_real_width_at_every_batch_size(hidden, heads, inter, layers):
    """The tiny configurations never reach the kernels that wide layers get at 17 to 64 tokens (k ranges
    split over blocks, large tiles for few rows, a rotation kernel of its own after the qkv product).
    One layer of an 8B and of a 70B model's widths, and two of a 1B model's (narrow weights with long rows get blocks of their
    own, and what the second layer's first norm needs is left by the first layer's last product): the same decoded token alone,
    among 8, 24 and 48 requests and beside a prompt portion, in float32 and bfloat16, against the plain implementation run on
    the tensors the engine gives back."""
    from llm_rs_amd import LlamaConfig
    cfg = LlamaConfig.from_dict(dict(
        architectures=["LlamaForCausalLM"], num_hidden_layers=layers, hidden_size=hidden, num_attention_heads=heads,
        num_key_value_heads=8, head_dim=hidden // heads, intermediate_size=inter, vocab_size=2000, rope_theta=500000.0,
        max_position_embeddings=4096, rms_norm_eps=1e-5, tie_word_embeddings=True))
    n_req, plen = 48, 24
    prompts = [random_tokens(2000, plen + 1, seed=300 + i) for i in range(n_req)]
    portion = random_tokens(2000, 150, seed=399)
    rows, weights = {}, None
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_random(cfg, 5, dtype=dtype, page_size=16, num_pages=256, max_requests=64)
        if weights is None:
            weights = {n: t.double() for n, t in eng.weights().items()}     # made on the device, read back
        slots = [eng.open_request() for _ in range(n_req)]
        for s, p in zip(slots, prompts):
            eng.step([StepEntry(s, 0, p[:plen], [])])
        extra = eng.open_request()
        decode = lambda n: [StepEntry(slots[i], plen, [prompts[i][plen]], [0]) for i in range(n)]
        got = {n: eng.step(decode(n)).float().cpu().clone() for n in (1, 8, 24, 48)}
        got["mixed"] = eng.step(decode(20) + [StepEntry(extra, 0, portion, [len(portion) - 1])]).float().cpu().clone()
        rows[dtype] = got
        del eng
    checked = [0, 7, 19, 23, 47]                                            # requests whose rows the plain implementation computes
    plain = {i: plain_forward(cfg.to_dict(), weights, prompts[i])[-1] for i in checked}
    plain_portion = plain_forward(cfg.to_dict(), weights, portion)[-1]
    scale = max(logit_scale(r) for r in plain.values())
    for dtype in ("float32", "bfloat16"):
        allowed = tolerance_for(dtype, cfg.to_dict(), {n: t.bfloat16() if t.dim() > 1 else t.float() for n, t in weights.items()},
                                [prompts[i] for i in checked[:3]] + [portion])
        worst = 0.0
        for key, got in rows[dtype].items():
            n = min(len(got), n_req) if key != "mixed" else 20
            for i in (i for i in checked if i < n):
                err = float((got[i].double() - plain[i]).abs().max()) / scale
                assert err <= allowed, f"{dtype} batch {key}, request {i}: error {err:.3e} of the largest logit, allowed {allowed:.3e}"
                worst = max(worst, err)
        err = float((rows[dtype]["mixed"][20].double() - plain_portion).abs().max()) / logit_scale(plain_portion)
        assert err <= allowed, f"{dtype}: prompt portion beside decoded tokens: {err:.3e}, allowed {allowed:.3e}"
        note(dtype, max(worst, err))
        if dtype == "bfloat16":
            note("bfloat16, of what is allowed", max(worst, err) / allowed)


def test_requests_that_come_and_go(folders):
    """Requests submitted while others are running, one cancelled on its way: every output equals
    the request generated alone, and all pages and slots come back."""
    which = "B"
    cfg, _ = read_model_folder(folders[which])
    prompts = [random_tokens(cfg["vocab_size"], n, seed=400 + n) for n in (40, 3, 150, 21, 9, 77)]
    kw = dict(temperature=0.9, top_k=50, top_p=0.95)
    limits = [30, 12, 18, 25, 40, 10]
    alone_eng = engine(folders[which], which, "float32")
    alone = [alone_eng.generate([p], max_new_tokens=m, seed=60 + i, **kw)[0] for i, (p, m) in enumerate(zip(prompts, limits))]
    eng = engine(folders[which], which, "float32", max_chunk=32, max_requests=4)     # fewer slots than requests: some wait for one
    arrivals = {0: [0, 1], 3: [2], 10: [3, 4], 11: [5]}                               # step -> prompts submitted before it
    number, got, reasons, step = {}, {}, {}, 0
    cancelled = None
    while step < 12 or eng.has_unfinished():
        for i in arrivals.get(step, []):
            number[eng.submit(prompts[i], limits[i], seed=60 + i, **kw)] = i
            got[i] = []
        if step == 14:                                  # prompt 2 is still running: take it out
            cancelled = [r for r, i in number.items() if i == 2][0]
            eng.cancel(cancelled)
        for e in eng.advance():
            assert e.request != cancelled
            if e.token is not None:
                got[number[e.request]].append(e.token)
            if e.finished:
                reasons[number[e.request]] = e.finished
        step += 1
    for i in (0, 1, 3, 4, 5):
        assert got[i] == alone[i] and reasons[i] == "length", f"request {i}"
    assert 0 < len(got[2]) < limits[2] and got[2] == alone[2][:len(got[2])] and 2 not in reasons
    core = eng.cache.core
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0 and not eng.has_unfinished()
    assert eng.advance() == []


def test_bfloat16_under_preemption_follows_float32():
    """A model of middling width (1024 wide, 6 layers), 60 requests, a pool so small that requests are
    evicted and computed again, greedy in bfloat16: every chosen token is the float32 engine's choice
    for the same prefix, or so close to it that rounding decides."""
    import random
    from llm_rs_amd import LlamaConfig
    cfg = LlamaConfig.from_dict(dict(
        architectures=["LlamaForCausalLM"], num_hidden_layers=6, hidden_size=1024, num_attention_heads=16,
        num_key_value_heads=4, head_dim=64, intermediate_size=2816, vocab_size=5000, rope_theta=10000.0,
        max_position_embeddings=2048, rms_norm_eps=1e-5, tie_word_embeddings=False))
    rnd = random.Random(3)
    prompts = [random_tokens(5000, rnd.randint(1, 600), seed=500 + i) for i in range(60)]
    limits = [rnd.randint(1, 80) for _ in prompts]
    bf = Engine.from_random(cfg, 1, dtype="bfloat16", page_size=16, num_pages=70, max_requests=64, max_batch_tokens=512, max_chunk=64)
    out = bf.generate(prompts, max_new_tokens=limits)
    assert bf.last_stats.preemptions > 0, "the case must make the scheduler evict"
    core = bf.cache.core
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
    del bf
    ref = Engine.from_random(cfg, 1, dtype="float32", page_size=16, num_pages=64, max_requests=2)
    weights = {n: t.double() for n, t in ref.weights().items()}
    shortest = sorted(range(len(prompts)), key=lambda i: len(prompts[i]) + len(out[i]))[:3]
    allowed = tolerance_for("bfloat16", cfg.to_dict(), {n: t.bfloat16() if t.dim() > 1 else t.float() for n, t in weights.items()},
                            [prompts[i] + out[i] for i in shortest])
    for i, (p, o) in enumerate(zip(prompts, out)):
        assert len(o) == limits[i]
        slot = ref.open_request()
        logits = ref.step([StepEntry(slot, 0, p + o, list(range(len(p) - 1, len(p) + len(o) - 1)))]).float()
        ref.close_request(slot)
        if i in shortest:       # the float32 engine that judges here is itself judged by the plain implementation
            plain = plain_forward(cfg.to_dict(), weights, p + o)[len(p) - 1:len(p) + len(o) - 1]
            assert float((logits.double().cpu() - plain).abs().max()) <= TOLERANCE["float32"] * logit_scale(plain), i
        scale = logit_scale(logits)
        chosen = logits[torch.arange(len(o)), torch.tensor(o, device=logits.device)]
        gap = float((logits.max(dim=1).values - chosen).max()) / scale
        assert gap <= allowed, f"request {i}: a chosen token lies {gap:.3e} of the logit scale below the float32 choice (allowed {allowed:.3e})"


def test_a_dropped_engine_is_freed_at_once(folders):
    """No cycle of references holds an engine: when the last name for it goes, its device memory and its
    recorded graphs go too, without the cycle collector (which may run at any moment, and must not find
    such things to destroy while another engine records a graph)."""
    import gc
    import weakref
    gc.collect()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    gc.disable()
    try:
        eng = engine(folders["B"], "B", "bfloat16")
        eng.generate([[1, 2, 3, 4, 5]], max_new_tokens=12)
        assert eng.runner.graph_replays > 0, "the case must have recorded a graph"
        gone = [weakref.ref(eng), weakref.ref(eng.runner), weakref.ref(eng.cache), weakref.ref(eng.model)]
        del eng
        assert all(r() is None for r in gone)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() <= before
    finally:
        gc.enable()


def test_only_so_many_recorded_graphs_are_kept(folders):
    """More batch shapes than graphs may be kept: the least recently replayed one goes, comes back by being
    recorded again, and every step still equals the eager engine's."""
    which, dtype = "B", "bfloat16"
    cfg, _ = read_model_folder(folders[which])
    recorded, eager = engine(folders[which], which, dtype), engine(folders[which], which, dtype)
    eager.runner.use_graphs = False
    recorded.runner.max_graphs = 2
    seqs = [random_tokens(cfg["vocab_size"], 100, seed=600 + i) for i in range(4)]
    sr, se = [recorded.open_request() for _ in seqs], [eager.open_request() for _ in seqs]
    for i, seq in enumerate(seqs):
        for eng, sl in ((recorded, sr), (eager, se)):
            eng.step([StepEntry(sl[i], 0, seq[:10], [])])
    pos = [10] * 4
    for turn in range(6):
        for n in (4, 3, 2, 1):                       # four shapes, each seen three times in a row
            for _ in range(3):
                a = recorded.step([StepEntry(sr[i], pos[i], [seqs[i][pos[i]]], [0]) for i in range(n)]).clone()
                b = eager.step([StepEntry(se[i], pos[i], [seqs[i][pos[i]]], [0]) for i in range(n)]).clone()
                torch.cuda.synchronize()
                assert torch.equal(a, b)
                for i in range(n):
                    pos[i] += 1
            assert len(recorded.runner._graphs) <= 2
    assert recorded.runner.graph_replays > 20
