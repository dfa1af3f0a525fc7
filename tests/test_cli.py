"""The command line (src/cli/mod.rs:5-69, src/main.rs:84-151): random-weights mode and argument
errors here; a greedy completion through `bin/llm-rs` against the plain implementation on the GPU."""
import json
import os
import subprocess
import sys

import pytest
import torch

from llm_rs_amd import cli, load_config
from plain_llama import plain_generate, read_model_folder
from tiny_configs import TINY_A, TINY_B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "bin", "llm-rs")


def run(*args, **kw):
    return subprocess.run([sys.executable, PROGRAM, *args], capture_output=True, text=True, timeout=600, **kw)


def test_init_writes_a_model_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    out = tmp_path / "model"
    p = run("init", "--config", str(tmp_path / "config.json"), "--seed", "3", "--out", str(out))
    assert p.returncode == 0 and "Wrote" in p.stderr
    assert sorted(os.listdir(out)) == ["config.json", "model.safetensors"]
    cfg, weights = read_model_folder(str(out))
    assert load_config(str(out)).num_hidden_layers == 3 and weights["lm_head.weight"].shape == (384, 96)
    # the same seed gives the same file, another seed another
    p = run("init", "--config", str(tmp_path / "config.json"), "--seed", "3", "--out", str(tmp_path / "again"))
    assert open(out / "model.safetensors", "rb").read() == open(tmp_path / "again" / "model.safetensors", "rb").read()
    p = run("init", "--config", str(tmp_path / "config.json"), "--seed", "4", "--out", str(tmp_path / "other"))
    assert open(out / "model.safetensors", "rb").read() != open(tmp_path / "other" / "model.safetensors", "rb").read()


def test_argument_errors(tmp_path, capsys):
    assert cli.main(["complete", "-p", "1 2 3"]) == 1 and "--model is required" in capsys.readouterr().err
    assert cli.main(["-m", str(tmp_path), "chat"]) == 1 and "tokenizer" in capsys.readouterr().err
    assert cli.main(["-m", str(tmp_path), "serve", "-p", "8081"]) == 1 and "HTTP server" in capsys.readouterr().err
    with pytest.raises(SystemExit):
        cli.main(["-m", str(tmp_path)])                                   # no command
    assert cli.main(["-m", str(tmp_path), "complete"]) == 1 and "needs a prompt" in capsys.readouterr().err
    assert cli.main(["-m", str(tmp_path), "complete", "-p", "1", "--prompt-len", "4"]) == 1       # one or the other
    assert "needs a prompt" in capsys.readouterr().err
    assert cli.main(["--config", str(tmp_path / "c.json"), "complete", "-p", "1"]) == 1
    assert "--random-weights" in capsys.readouterr().err, "a configuration alone has no weights"
    args = cli.build_parser().parse_args(["--config", "c.json", "--random-weights", "5", "complete", "--prompt-ids", "1,2"])
    assert (args.config, args.random_weights, args.prompt, args.prompt_len) == ("c.json", 5, "1,2", None)
    args = cli.build_parser().parse_args(["-m", "x", "replay", "--out", "o", "--max-tokens", "128"])
    assert (args.command, args.out, args.max_tokens) == ("replay", "o", 128)
    assert cli.build_parser().parse_args(["-m", "x", "--dtype", "f32", "bench"]).dtype == "float32"
    assert cli.build_parser().parse_args(["-m", "x", "--dtype", "bf16", "bench"]).dtype == "bfloat16"
    args = cli.build_parser().parse_args(["-m", "x", "bench"])
    assert (args.prompt_len, args.batch, args.context) == (2048, 8, 2048)
    with pytest.raises(SystemExit, match="token ids"):
        cli.parse_ids("hello world")
    assert cli.parse_ids("1, 2  3,4") == [1, 2, 3, 4]
    capsys.readouterr()
    assert cli.main(["-m", str(tmp_path / "nothing"), "complete", "-p", "1"]) == 1
    assert capsys.readouterr().err.startswith("Error:")
    # the reference's defaults for sampling (src/cli/mod.rs:49-58) and for -n
    args = cli.build_parser().parse_args(["-m", "x", "complete", "-p", "1"])
    assert (args.temperature, args.top_k, args.top_p, args.seed, args.max_tokens) == (0.7, 40, 0.9, 42, 256)


def test_the_line_about_the_model_comes_from_the_configuration():
    from llm_rs_amd import LlamaConfig
    line = cli.describe_model(LlamaConfig.from_dict(TINY_A))
    assert line.startswith("LlamaForCausalLM: ") and "hidden_size=64" in line and "num_key_value_heads=2" in line and "vocab_size=256" in line

    class Other:
        def to_dict(self):
            return {"architectures": ["OtherForCausalLM"], "width": 5, "tied": True, "eps": 1e-5}
    assert cli.describe_model(Other()) == "OtherForCausalLM: width=5"


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16")])
def test_complete_on_the_gpu(tmp_path, which, dtype):
    (tmp_path / "config.json").write_text(json.dumps({"A": TINY_A, "B": TINY_B}[which]))
    folder = tmp_path / "model"
    assert run("init", "--config", str(tmp_path / "config.json"), "--seed", "9", "--out", str(folder)).returncode == 0
    cfg, weights = read_model_folder(str(folder))
    prompt = torch.randint(0, cfg["vocab_size"], (21,), generator=torch.Generator().manual_seed(3)).tolist()
    p = run("-m", str(folder), "--dtype", dtype, "--page-size", "4" if which == "A" else "16", "--num-pages", "64",
            "complete", "-p", " ".join(map(str, prompt)), "-n", "8", "--temperature", "0")
    assert p.returncode == 0, p.stderr[-2000:]
    got = [int(t) for t in p.stdout.split()]
    err = p.stderr
    for piece in ("Prompt tokens: 21", "Prefill: 21 tokens in", "Generated: 8 tokens in", "tok/s", "[gpu=", "overhead="):
        assert piece in err, err
    assert f"LlamaForCausalLM: " in err and f"hidden_size={cfg['hidden_size']}" in err
    if dtype == "float32":
        assert got == plain_generate(cfg, weights, prompt, 8)
    else:
        from test_generate_gpu import check_greedy_path
        check_greedy_path(cfg, weights, prompt, got, dtype)
    # sampling with the reference's defaults runs, and is the plain implementation's draw in 32-bit
    if dtype == "float32":
        p = run("-m", str(folder), "--dtype", dtype, "--page-size", "4" if which == "A" else "16", "--num-pages", "64",
                "complete", "-p", " ".join(map(str, prompt)), "-n", "6")
        assert p.returncode == 0, p.stderr[-2000:]
        assert [int(t) for t in p.stdout.split()] == plain_generate(cfg, weights, prompt, 6, temperature=0.7, top_k=40, top_p=0.9, seed=42)


@pytest.mark.gpu
def test_random_weights_from_the_command_line_are_the_folders(tmp_path):
    """`--config FILE --random-weights SEED` makes on the device the tensors that `init --seed SEED` writes: the same
    completion either way, with a prompt given as ids and with `--prompt-len`; and `replay` is bin/trace_run."""
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    folder = tmp_path / "model"
    assert run("init", "--config", str(tmp_path / "config.json"), "--seed", "4", "--out", str(folder)).returncode == 0
    common = ("--dtype", "float32", "--num-pages", "64")
    a = run("-m", str(folder), *common, "complete", "--prompt-len", "19", "-n", "7", "--seed", "3")
    b = run("--config", str(tmp_path / "config.json"), "--random-weights", "4", *common, "complete", "--prompt-len", "19", "-n", "7", "--seed", "3")
    assert a.returncode == 0 and b.returncode == 0, a.stderr[-1500:] + b.stderr[-1500:]
    assert a.stdout == b.stdout and len(a.stdout.split()) == 7 and "Prompt tokens: 19" in b.stderr
    cfg, weights = read_model_folder(str(folder))
    prompt = torch.randint(0, cfg["vocab_size"], (19,), generator=torch.Generator().manual_seed(3)).tolist()
    assert [int(t) for t in a.stdout.split()] == plain_generate(cfg, weights, prompt, 7, temperature=0.7, top_k=40, top_p=0.9, seed=3)
    # replay: the same files as the program bin/trace_run writes
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:11], "want": [0, 10]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[11:], "want": [7]}, {"id": "b", "tokens": prompt[:5], "want": []}], "end": ["a", "b"]}]
    text = "".join(json.dumps(st) + "\n" for st in steps)
    p = run("--config", str(tmp_path / "config.json"), "--random-weights", "4", "--dtype", "float32", "replay",
            "--out", str(tmp_path / "r1"), "--max-tokens", "128", input=text)
    assert p.returncode == 0 and p.stdout.split() == ["done", "0", "done", "1"], p.stderr[-1500:]
    q = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32",
                        "--out", str(tmp_path / "r2"), "--max-tokens", "128"], input=text, capture_output=True, text=True, timeout=600)
    assert q.returncode == 0, q.stderr[-1500:]
    for name in ("0.f32", "1.f32"):
        assert open(tmp_path / "r1" / name, "rb").read() == open(tmp_path / "r2" / name, "rb").read()
    import numpy as np
    got = torch.from_numpy(np.fromfile(tmp_path / "r1" / "1.f32", dtype="<f4")).double()
    from plain_llama import plain_forward
    want = plain_forward(cfg, weights, prompt)[18]
    assert float((got - want).abs().max()) <= 3e-5 * float(want.abs().max())


@pytest.mark.gpu
def test_bench_subcommand_and_the_table_by_kernel(tmp_path):
    """`bench` prints its figures; with LLM_PERF set (the reference's switch, src/backend/metal/mod.rs:235,321-400)
    every kernel call is timed by itself, steps are not recorded into graphs, and a table by kernel follows on
    stderr: every kind of kernel the step runs has a row with calls, time and what it moved or computed, and the
    tokens are those of the run without the switch."""
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    base = ("--config", str(tmp_path / "config.json"), "--random-weights", "2", "--num-pages", "64")
    p = run(*base, "bench", "--prompt-len", "64", "--batch", "3", "--context", "48", "--steps", "5")
    assert p.returncode == 0, p.stderr[-1500:]
    line = json.loads(p.stdout.strip().splitlines()[-1])
    assert line["prefill_tokens"] == 64 and line["decode_batch"] == 3 and line["prefill_tok_s"] > 0 and line["decode_tok_s"] > 0
    for dtype in ("bfloat16", "float32"):
        for sampling in (("--temperature", "0"), ()):
            plain = run(*base, "--dtype", dtype, "complete", "--prompt-len", "40", "-n", "12", *sampling)
            timed = run(*base, "--dtype", dtype, "complete", "--prompt-len", "40", "-n", "12", *sampling, env={**os.environ, "LLM_PERF": "1"})
            assert plain.returncode == 0 and timed.returncode == 0, plain.stderr[-1500:] + timed.stderr[-1500:]
            assert timed.stdout == plain.stdout, "timing each kernel (and running every step eagerly) must not change the tokens"
            assert "TOTAL" not in plain.stderr
            rows = {}
            for ln in timed.stderr.splitlines():
                m = __import__("re").match(r"\s{2}(\S.*?)\s{2,}(\d+)\s+([\d.]+)(ms|us)\s+([\d.]+)%\s+(\d+) \(\s*[\d.]+%\)\s+(.*)$", ln)
                if m and m.group(1) != "TOTAL":
                    rows[m.group(1)] = (int(m.group(2)), float(m.group(3)), int(m.group(6)), m.group(7).strip())
            kinds = {name.split()[0] for name in rows}
            want = {"embed", "gemm", "attention", "argmax" if sampling else "sample"}
            assert want <= kinds, (kinds, timed.stderr[-3000:])
            assert "TOTAL" in timed.stderr
            assert all(calls > 0 and t > 0 for calls, t, _, _ in rows.values())
            gemms = {n: r for n, r in rows.items() if n.startswith("gemm")}
            # (a kernel's first call waits for its code to reach the device, so a label that ran once may show 0 GB/s)
            assert all(r[3] != "-" for r in gemms.values()) and any(r[2] > 0 for r in gemms.values()), "a product has bytes and operations"
            # 13 steps (one prompt step, 12 decode steps less the last) of 3 layers: each layer's products are counted
            assert sum(r[0] for r in gemms.values()) >= 12 * (3 * 4 + 1)
