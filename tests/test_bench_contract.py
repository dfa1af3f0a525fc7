"""bench.py's contract where no GPU is needed: more than one GPU is refused in one line with exit
code 2, and each workload's line has the keys the record keeps, with a flat `config` of at most 20 keys."""
import importlib.util
import json
import os
import subprocess
import sys
from types import SimpleNamespace

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

REQUIRED = {"metric": str, "value": float, "unit": str, "n_gpus": int, "steps": int, "warmup": int, "ms_per_step": float,
            "higher_is_better": bool, "scaling": str, "dtype": str, "data": str, "config": dict}


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def check_line(line):
    line = json.loads(json.dumps(line))                  # what the record keeps is what JSON keeps
    for key, kind in REQUIRED.items():
        assert key in line and isinstance(line[key], (kind, int) if kind is float else kind), key
    assert "vs_baseline" in line and line["n_gpus"] == 1 and line["higher_is_better"] is True
    cfg = line["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values()), "flat, at most 20 keys"
    for key in ("model", "global_batch", "seq_len", "parallelism", "layers_run", "layers_of_config", "hidden_size",
                "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size", "vocab_size", "page_size"):
        assert key in cfg, key
    return line


def test_more_than_one_gpu_is_refused_in_one_line():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 2
    lines = [l for l in run.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_lines_of_every_workload():
    b = load_bench()
    args = SimpleNamespace(batch=8, context=2048, steps=64, warmup=8, prefill_tokens=2048, dtype="bfloat16", new_tokens=256)
    host = b.host_share(4.0e-3, 3.9e-3)
    assert host == {"wall_ms_per_step": 4.0, "device_ms_per_step": 3.9, "overhead_frac": 0.025}
    line = check_line(b.decode_line(args, 32, 4.0e-3, 15.0e9, 131072, 33e-3, {"decode_b1": 270.0, "decode_b64": 7300.0}, host))
    assert line["value"] == 2000.0 and line["config"]["layers_run"] == line["config"]["layers_of_config"] == 32
    assert set(line["prefill"]) == {"value", "tokens", "ms", "frac"} and line["prefill"]["tokens"] == 2048
    assert set(line["roofline"]) == {"bound", "achieved", "peak", "unit", "frac"} and line["roofline"]["bound"] == "hbm"
    assert line["roofline"]["peak"] == 8000.0 and abs(line["roofline"]["frac"] - line["roofline"]["achieved"] / 8000.0) < 1e-3
    # bytes of the step: every weight once and the cache of the live requests, as the record's reader recomputes them
    want = (15.0e9 + 8 * (2048 + 8 + 32) * 131072) / 4.0e-3 / 1e9
    assert abs(line["roofline"]["achieved"] - want) < 0.1
    assert set(line["points"]) == {"decode_b1", "decode_b64"} and line["host"]["overhead_frac"] == 0.025
    # prefill operations of the 8B shape at 2,048 tokens: 29.7 TFLOP
    assert abs(b.prefill_flops(b.LLAMA_8B, 32, 2048) / 1e12 - 29.69) < 0.05

    line = check_line(b.serve_line(args, 16, 256, 543071, 65536, 3.9, 538, 3.5, 0, 2048))
    assert line["config"]["model"] == "Llama-3.2-1B shape" and line["config"]["global_batch"] == 256
    assert abs(line["value"] - 65536 / 3.9) < 0.1 and abs(line["total_tokens_per_s"] - (543071 + 65536) / 3.9) < 0.1
    assert 0.0 < line["host"]["overhead_frac"] < 0.2

    args.steps, args.warmup = 8, 2
    line = check_line(b.mixed_line(args, 80, 0.34, 141e9, 22e9, b.host_share(0.34, 0.339)))
    assert line["config"]["layers_run"] == 80 and line["config"]["decodes"] == 16 and line["config"]["prefill_chunk"] == 2048
    assert abs(line["value"] - 2064 / 0.34) < 0.1 and line["compute"]["unit"] == "TFLOP/s" and 0 < line["compute"]["frac"] < 1

    line = check_line(b.sizes_line(args, 32, {"decode_b1_ctx8192": 250.0, "decode_b256_ctx2048": 15000.0},
                                   {"decode_b1_ctx8192": 0.5, "decode_b256_ctx2048": 0.4}))
    assert set(line["points"]) == set(line["roofline_frac"])
    line = check_line(b.sizes_line(args, 16, {"decode_b1_ctx2048": 900.0}, {"decode_b1_ctx2048": 0.4}, 0.0011, "Llama-3.2-1B shape"))
    assert line["config"]["model"] == "Llama-3.2-1B shape" and line["config"]["hidden_size"] == 2048 and "1B shape" in line["metric"]
    line = check_line(b.long_line(args, 32, {"decode_b1_ctx131008": 130.0, "decode_b4_ctx32704": 400.0},
                                  {"decode_b1_ctx131008": 0.6, "decode_b4_ctx32704": 0.6}, 0.0077))
    assert line["config"]["max_context"] == 131072 and set(line["points"]) == set(line["roofline_frac"])
    line = check_line(b.prompts_line(args, 32, {"prefill_2048": 67000.0, "prefill_2049": 60000.0}, {"prefill_2048": 0.39, "prefill_2049": 0.35}, 0.0305))
    assert set(line["points"]) == set(line["peak_frac"]) and line["value"] == 67000.0 and abs(line["ms_per_step"] - 30.5) < 1e-6


import pytest


@pytest.mark.gpu
def test_the_default_workload_runs_and_fills_its_line():
    """The default workload with one layer and a few steps, in this process: decode steps go through the engine's own
    loop (every call gives every request a token, or the run stops), and the line carries a prefill, a roofline,
    both points and the host's share."""
    bench = load_bench()
    args = SimpleNamespace(gpus=1, steps=6, warmup=4, workload="decode8b", batch=8, context=300, prefill_tokens=256, layers=1,
                           dtype="bfloat16", points="1,20,3@700", only="", requests=0, new_tokens=0, max_batch_tokens=2048)
    line = check_line(bench.run_decode8b(args))
    assert line["value"] > 0 and abs(line["value"] - 8 / (line["ms_per_step"] * 1e-3)) <= 1e-3 * line["value"]
    assert line["config"]["layers_run"] == 1 and line["config"]["layers_of_config"] == 32 and line["config"]["global_batch"] == 8
    assert set(line["points"]) == {"decode_b1", "decode_b20", "decode_b3_ctx700"} and all(v > 0 for v in line["points"].values())
    assert set(line["points_frac"]) == set(line["points"]) and all(0 < v < 1 for v in line["points_frac"].values())
    assert line["metric"].endswith("prefill tok/s at 256 tokens and batch 1/20 alongside")
    assert line["prefill"]["tokens"] == 256 and 0 < line["prefill"]["frac"] < 1
    assert line["roofline"]["bound"] == "hbm" and 0 < line["roofline"]["frac"] < 1
    assert 0 <= line["host"]["overhead_frac"] < 0.5 and line["host"]["device_ms_per_step"] > 0
