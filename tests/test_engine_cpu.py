"""The engine's host side with the emulated kernels in place of the device:
requests that come and go through submit/advance, a request that can never run,
export of the model's tensors, the seeded fill, and the order of checks at start."""
import numpy as np
import pytest
import torch

from emulated_kernels import EmulatedKernels
from llm_rs_amd import Engine, KernelError, LlamaConfig, random_model_tensors, use_kernels, write_model_folder
from llm_rs_amd.weights import fill_normal
from plain_llama import plain_generate
from tiny_configs import TINY_A, TINY_B


@pytest.fixture
def engine_a():
    cfg = LlamaConfig.from_dict(TINY_A)
    tensors = random_model_tensors(cfg, 4)
    with use_kernels(EmulatedKernels()):
        yield Engine(cfg, tensors, dtype="float32", device="cpu", page_size=4, num_pages=24, max_requests=3), tensors


def test_a_request_that_can_never_run_is_refused_at_submit_and_blocks_nobody(engine_a):
    eng, tensors = engine_a
    prompts = [[5, 6, 7], [9, 1], [3, 3, 3, 3]]
    got, ids = {}, []
    ids.append(eng.submit(prompts[0], 5))
    with pytest.raises(ValueError, match="positions"):
        eng.submit(list(range(100)), 60)                    # 160 positions, the model has 128
    with pytest.raises(ValueError, match="pages"):
        eng.submit(list(range(90)), 20)                     # 28 pages at once, the pool has 24
    ids += [eng.submit(p, 5) for p in prompts[1:]]
    assert ids == [0, 1, 2], "a refused request takes no number and leaves nothing behind"
    while eng.has_unfinished():
        for e in eng.advance():
            got.setdefault(e.request, []).append(e.token)
    cfg = TINY_A
    for r, p in zip(ids, prompts):
        assert got[r] == plain_generate(cfg, tensors, p, 5)
    core = eng.cache.core
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0


@pytest.mark.parametrize("which,dtype", [("A", "bfloat16"), ("B", "float32"), ("B", "bfloat16")])
def test_weights_gives_back_what_was_loaded(which, dtype):
    cfg = LlamaConfig.from_dict({"A": TINY_A, "B": TINY_B}[which])
    tensors = random_model_tensors(cfg, 11)
    with use_kernels(EmulatedKernels()):
        eng = Engine(cfg, tensors, dtype=dtype, device="cpu", page_size=4, num_pages=8, max_requests=2)
    back = eng.weights()
    assert sorted(back) == sorted(tensors)
    for name, t in tensors.items():
        want = t.float() if dtype == "float32" or name.endswith("norm.weight") else t
        assert back[name].dtype == want.dtype and torch.equal(back[name], want), name
    # and what comes back can be loaded again
    with use_kernels(EmulatedKernels()):
        again = Engine(cfg, back, dtype=dtype, device="cpu", page_size=4, num_pages=8, max_requests=2)
        assert again.generate([[1, 2, 3]], max_new_tokens=4) == eng.generate([[1, 2, 3]], max_new_tokens=4)


def test_seeded_fill_is_a_function_of_key_and_index():
    a = fill_normal(torch.empty(100003), 77, 0.0, 1.0)
    b = fill_normal(torch.empty(100003), 77, 0.0, 1.0)
    c = fill_normal(torch.empty(100003), 78, 0.0, 1.0)
    assert torch.equal(a, b) and not torch.equal(a, c)
    # a longer tensor of the same key starts with the same values: element i depends on (key, i) alone,
    # however the range was shared out over threads
    long = fill_normal(torch.empty(400000), 77, 0.0, 1.0)
    assert torch.equal(long[:100003], a)
    # bfloat16 is the float32 value rounded once, to nearest even
    h = fill_normal(torch.empty(100003, dtype=torch.bfloat16), 77, 0.0, 1.0)
    assert torch.equal(h, a.bfloat16())
    shifted = fill_normal(torch.empty(1000), 77, 1.0, 0.1)
    assert float((shifted - (1.0 + 0.1 * a[:1000])).abs().max()) < 2e-7      # one fused multiply-add


def test_seeded_fill_is_normal():
    z = fill_normal(torch.empty(4_000_000), 2024, 0.0, 1.0).double()
    assert abs(float(z.mean())) < 2e-3 and abs(float(z.var()) - 1.0) < 4e-3
    assert abs(float((z ** 3).mean())) < 1e-2 and abs(float((z ** 4).mean()) - 3.0) < 3e-2
    for bound, mass in ((1.0, 0.317311), (2.0, 0.045500), (3.0, 0.002700)):
        assert abs(float((z.abs() > bound).double().mean()) - mass) < 0.02 * mass + 1e-4
    assert abs(float((z[1:] * z[:-1]).mean())) < 2e-3, "neighbours are uncorrelated"
    assert float(z.abs().max()) < 5.8                      # u1 >= 2^-24: sqrt(48 ln 2) = 5.77


def test_no_gpu_is_said_before_any_weight_is_read(tmp_path, monkeypatch):
    """Without a GPU (or a kernel library) the engine says so first: a folder of many gigabytes is
    not read only to find that out."""
    if torch.cuda.is_available():
        pytest.skip("this machine has a GPU")
    cfg = LlamaConfig.from_dict(TINY_A)
    write_model_folder(str(tmp_path), cfg, random_model_tensors(cfg, 0))
    import llm_rs_amd.engine.engine as engine_module
    read = []
    monkeypatch.setattr(engine_module, "load_tensors", lambda *a, **k: read.append(1))
    with pytest.raises(Exception, match="GPU|gfx950|kernel"):
        Engine.from_folder(str(tmp_path))
    assert read == []


@pytest.mark.parametrize("which", ["A", "B"])
def test_a_step_started_before_the_last_one_is_read_changes_no_output(which):
    """`overlap` (a step is planned and started while the step before is in flight, its samples handed over on the
    device) against stepping in turn: the same tokens and finish reasons, with stop tokens, sampling with a
    temperature, requests that end at different times and a pool so small that requests give way."""
    cfg_d = TINY_A if which == "A" else TINY_B
    cfg = LlamaConfig.from_dict(cfg_d)
    tensors = random_model_tensors(cfg, 11)
    rng = np.random.default_rng(5)
    prompts = [rng.integers(0, cfg.vocab_size, int(n)).tolist() for n in (3, 17, 9, 1, 26, 12, 5)]
    limits = [16, 14, 1, 16, 6, 2, 15]
    seeds = [3, 4, 5, 6, 7, 8, 9]

    def run(overlap, temperature, stop):
        eng = Engine(cfg, tensors, dtype="float32", device="cpu", page_size=4, num_pages=10, max_requests=3,
                     max_batch_tokens=16, overlap=overlap)
        got = eng.generate(prompts, limits, temperature=temperature, top_k=20, top_p=0.95, seed=seeds,
                           stop_token_ids=stop, return_reasons=True)
        core = eng.cache.core
        assert core.pages_free() == 10 and core.slots_in_use() == 0 and not core.in_flight() and not eng.has_unfinished()
        return [(f.tokens, f.reason) for f in got], eng.last_stats

    with use_kernels(EmulatedKernels()):
        free, stats = run(False, 0.9, [])
        assert stats.preemptions > 0, "the case itself: the pool is too small for what three requests grow to"
        assert run(True, 0.9, [])[0] == free
        assert run(True, 0.0, [])[0] == run(False, 0.0, [])[0]
        # a stop token that does occur in the middle of an output: a token some request sampled that it had not before
        i, at = next((i, j) for i, (toks, _) in enumerate(free) for j in range(1, len(toks)) if toks[j] not in toks[:j])
        stop = [free[i][0][at]]
        in_turn = run(False, 0.9, stop)[0]
        assert in_turn[i] == (free[i][0][:at], "stop")
        assert run(True, 0.9, stop)[0] == in_turn


def test_cancel_while_a_step_is_in_flight(engine_a):
    eng, tensors = engine_a
    assert eng.overlap
    a = eng.submit([5, 6, 7], 8)
    b = eng.submit([9, 1], 8)
    got = {a: [], b: []}
    for e in eng.advance():                    # the first call starts two steps and lands the first
        got[e.request].append(e.token)
    assert eng.cache.core.in_flight()
    eng.cancel(a)                              # a has an entry in the step in flight
    c = eng.submit([3, 3, 3, 3], 4)            # takes a's slot
    got[c] = []
    while eng.has_unfinished():
        for e in eng.advance():
            got[e.request].append(e.token)
    assert got[b] == plain_generate(TINY_A, tensors, [9, 1], 8)
    assert got[c] == plain_generate(TINY_A, tensors, [3, 3, 3, 3], 4), "what a's step in flight sampled is nobody's"
    assert len(got[a]) == 1
    core = eng.cache.core
    assert core.pages_free() == 24 and core.slots_in_use() == 0 and not core.in_flight()


@pytest.mark.parametrize("when", ["before the scheduler is told", "after the scheduler is told"])
@pytest.mark.parametrize("at_step", [1, 3, 6])
def test_an_interrupt_while_a_step_lands_leaves_engine_and_scheduler_agreeing(engine_a, when, at_step):
    """generate() is interrupted inside the landing of a step, once before the scheduler has taken the step's
    samples and once right after, with another step already started ahead.  The interrupt itself comes out (not an
    error about a step nobody knows), nothing is left held, and the engine generates the same tokens afterwards."""
    eng, tensors = engine_a
    assert eng.overlap
    core = eng.cache.core
    real, calls = core.commit, [0]

    def commit(sampled):
        calls[0] += 1
        if calls[0] == at_step and when.startswith("before"):
            raise KeyboardInterrupt
        finished = real(sampled)
        if calls[0] == at_step:
            raise KeyboardInterrupt
        return finished

    prompts = [[5, 6, 7], [9, 1], [3, 3, 3, 3, 8, 2, 1]]
    core.commit = commit
    try:
        with pytest.raises(KeyboardInterrupt):
            eng.generate(prompts, max_new_tokens=6)
    finally:
        core.commit = real
    assert calls[0] >= at_step
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
    assert not core.in_flight() and not eng.has_unfinished() and core.idle()
    got = eng.generate(prompts, max_new_tokens=6)
    assert got == [plain_generate(TINY_A, tensors, p, 6) for p in prompts]
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0 and not core.in_flight()
