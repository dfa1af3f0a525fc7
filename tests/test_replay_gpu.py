"""Replay on the GPU, through the real kernels, in 32-bit and bfloat16: each
request alone and whole; most of it in one step and the last 32 tokens one by
one; portions of changing size; and mixed, up to four live requests with so few
pages that they are used again.  Every wanted row is compared with the plain
implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from llm_rs_amd.engine.trace import TraceReplayer
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole
from plain_llama import read_model_folder
from replay_checks import check_rows, reference_rows, run_trace, tolerance_for
from tiny_configs import CONFIGS, PAGE_SIZE, make_folder

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 33, 100, 128], "B": [1, 7, 64, 130, 300]}


@pytest.fixture(scope="module")
def setup(tmp_path_factory):
    d = tmp_path_factory.mktemp("models")
    folders = {w: make_folder(d, w, seed=5) for w in "AB"}
    requests = {w: {f"r{i}": random_tokens(CONFIGS[w]["vocab_size"], n, seed=20 + i) for i, n in enumerate(LENGTHS[w])}
                for w in "AB"}
    reference = {w: reference_rows(folders[w], requests[w]) for w in "AB"}
    return folders, requests, reference


@pytest.fixture(scope="module")
def allowed(setup):
    """(model, dtype) -> how far from the plain implementation a row may be."""
    folders, requests, reference = setup
    out = {}
    for w in "AB":
        cfg, weights = read_model_folder(folders[w])
        for dtype in ("float32", "bfloat16"):
            out[w, dtype] = tolerance_for(dtype, cfg, weights, list(requests[w].values()), list(reference[w].values()))
    return out


CASES = [("A", "float32"), ("A", "bfloat16"), ("B", "float32"), ("B", "bfloat16")]


def _make(folder, which, dtype):
    return lambda n: TraceReplayer(folder, dtype, n, page_size=PAGE_SIZE[which], device="cuda")


def _check_clean(rep):
    core = rep.engine.cache.core
    assert core.pages_free() == core.pages_total() and core.slots_in_use() == 0


@pytest.mark.parametrize("which,dtype", CASES)
def test_whole(setup, allowed, which, dtype):
    folders, requests, reference = setup
    rows, rep = run_trace(_make(folders[which], which, dtype), whole(requests[which]))
    print("worst", check_rows(rows, reference[which], dtype, requests[which], allowed[which, dtype]))
    _check_clean(rep)


@pytest.mark.parametrize("which,dtype", CASES)
def test_last_32_one_by_one(setup, allowed, which, dtype):
    folders, requests, reference = setup
    rows, rep = run_trace(_make(folders[which], which, dtype), tail_decoded(requests[which], 32))
    check_rows(rows, reference[which], dtype, requests[which], allowed[which, dtype])
    _check_clean(rep)


@pytest.mark.parametrize("which,dtype", CASES)
def test_portions(setup, allowed, which, dtype):
    folders, requests, reference = setup
    rows, rep = run_trace(_make(folders[which], which, dtype), portions(requests[which]))
    check_rows(rows, reference[which], dtype, requests[which], allowed[which, dtype])
    _check_clean(rep)


@pytest.mark.parametrize("which,dtype", CASES)
def test_mixed_with_reused_pages(setup, allowed, which, dtype):
    folders, requests, reference = setup
    steps = mixed(requests[which], live=4)
    need = live_token_need(steps)
    total = sum(-(-len(t) // 64) * 64 for t in requests[which].values())
    assert need < total, "the pool must be too small to hold all requests at once, so that pages are used again"
    rows, rep = run_trace(_make(folders[which], which, dtype), steps, max_tokens=need)
    check_rows(rows, reference[which], dtype, requests[which], allowed[which, dtype])
    _check_clean(rep)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(setup, allowed, tmp_path, dtype):
    """bin/trace_run as a user calls it: JSON lines in, <step>.f32 files and `done` lines out."""
    folders, requests, reference = setup
    which = "B"
    steps = mixed(requests[which], live=3)
    out_dir = tmp_path / f"out_{dtype}"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folders[which], "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", str(live_token_need(steps))],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    vocab = CONFIGS[which]["vocab_size"]
    outputs = []
    for s in steps:
        n = sum(len(e["want"]) for e in s["entries"])
        f = out_dir / f"{s['step']}.f32"
        outputs.append(torch.from_numpy(np.fromfile(f, dtype="<f4").reshape(n, vocab).copy()) if n else None)
    check_rows(collect(steps, outputs), reference[which], dtype, requests[which], allowed[which, dtype])


# ---- one layer of an 8B model's widths ------------------------------------------------
@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    d = tmp_path_factory.mktemp("wide")
    folder = make_folder(d, "W", seed=9)
    requests = {f"w{i}": random_tokens(CONFIGS["W"]["vocab_size"], n, seed=40 + i) for i, n in enumerate([40, 100, 230, 70])}
    reference = reference_rows(folder, requests)
    cfg, weights = read_model_folder(folder)
    bound = {dtype: tolerance_for(dtype, cfg, weights, list(requests.values()), list(reference.values())) for dtype in ("float32", "bfloat16")}
    return folder, requests, reference, bound


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_wide_layer(wide, dtype, cut):
    """The four ways of cutting, on a layer as wide as an 8B model's, against the plain implementation."""
    folder, requests, reference, bound = wide
    steps = {"whole": lambda: whole(requests), "tail": lambda: tail_decoded(requests, 32),
             "portions": lambda: portions(requests), "mixed": lambda: mixed(requests, live=4)}[cut]()
    rows, rep = run_trace(_make(folder, "W", dtype), steps)
    print("worst", check_rows(rows, reference, dtype, requests, bound[dtype]))
    _check_clean(rep)
