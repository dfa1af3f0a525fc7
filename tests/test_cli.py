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
    with pytest.raises(SystemExit):
        cli.main(["-m", str(tmp_path), "complete"])                       # no prompt
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
