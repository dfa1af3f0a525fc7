"""The replay regimes on the engine's host logic (cache manager, batch builder,
step function), with the emulated kernels in place of the device."""
import pytest

from emulated_kernels import EmulatedKernels
from llm_rs_amd import use_kernels
from llm_rs_amd.engine.trace import TraceReplayer
from replay_cases import mixed, portions, random_tokens, tail_decoded, whole
from replay_checks import check_rows, reference_rows, run_trace, tolerance_for
from plain_llama import read_model_folder
from tiny_configs import CONFIGS, PAGE_SIZE, make_folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    d = tmp_path_factory.mktemp("models")
    return {w: make_folder(d, w, seed=3) for w in "AB"}


@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16")])
def test_regimes_agree_with_plain(folders, which, dtype):
    vocab = CONFIGS[which]["vocab_size"]
    lengths = {"A": [5, 17, 33, 40], "B": [1, 7, 64, 70]}[which]
    requests = {f"r{i}": random_tokens(vocab, n, seed=10 + i) for i, n in enumerate(lengths)}
    reference = reference_rows(folders[which], requests)
    cfg, weights = read_model_folder(folders[which])
    allowed = tolerance_for(dtype, cfg, weights, list(requests.values()), list(reference.values()))
    with use_kernels(EmulatedKernels()):
        make = lambda n: TraceReplayer(folders[which], dtype, n, page_size=PAGE_SIZE[which], device="cpu")
        for steps in (whole(requests), tail_decoded(requests, 8), portions(requests), mixed(requests)):
            rows, rep = run_trace(make, steps)
            check_rows(rows, reference, dtype, requests, allowed)
            core = rep.engine.cache.core
            assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0
