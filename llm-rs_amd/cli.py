"""Command line in the reference's manner (src/cli/mod.rs:5-69, src/main.rs:84-151):

    llm-rs -m MODEL_DIR complete -p "1 15 27 3" [-n 256] [--temperature 0.7 --top-k 40 --top-p 0.9 --seed 42]
    llm-rs init --config config.json --seed 0 --out MODEL_DIR        (random-weights mode)

`-m/--model` is a folder with config.json and model.safetensors (the reference
takes a GGUF file).  There is no tokenizer in this engine, so the prompt is
token ids, separated by spaces or commas, and the completion is printed as ids.
The statistics lines on stderr are the reference's: prompt tokens, prefill
tokens a second, generated tokens a second.  `chat` and `serve` need a tokenizer
and an HTTP server, which this engine does not have; they say so and exit.
"""
from __future__ import annotations

import argparse
import json
import re
import sys
import time
from typing import List


def _add_sampling(p: argparse.ArgumentParser) -> None:
    # defaults of the reference's SamplingArgs (src/cli/mod.rs:49-58)
    p.add_argument("--temperature", type=float, default=0.7)
    p.add_argument("--top-k", type=int, default=40)
    p.add_argument("--top-p", type=float, default=0.9)
    p.add_argument("--seed", type=int, default=42)


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="llm-rs", description="LLM inference on MI355X")
    ap.add_argument("-m", "--model", help="model folder (config.json + model.safetensors)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=None, help="KV pages (default: sized from free memory)")
    ap.add_argument("--max-batch-tokens", type=int, default=2048,
                    help="tokens a step may run (the reference's MAX_TOKENS_PER_STEP); longer prompts are cut into portions")
    sub = ap.add_subparsers(dest="command", required=True)
    c = sub.add_parser("complete", help="Single-shot completion of a prompt given as token ids")
    c.add_argument("-p", "--prompt", required=True, help="token ids, e.g. \"1 15 27\"")
    c.add_argument("-n", "--max-tokens", type=int, default=256)
    c.add_argument("--stop", default="", help="token ids that end the completion (default: eos_token_id of the config)")
    _add_sampling(c)
    ch = sub.add_parser("chat", help="(not available: needs a tokenizer)")
    ch.add_argument("-s", "--system", default=None)
    _add_sampling(ch)
    sv = sub.add_parser("serve", help="(not available: no HTTP server in this engine)")
    sv.add_argument("-p", "--port", type=int, default=8080)
    i = sub.add_parser("init", help="Write a model folder with random weights")
    i.add_argument("--config", required=True, help="a config.json")
    i.add_argument("--seed", type=int, default=0)
    i.add_argument("--out", required=True)
    i.add_argument("--weights-dtype", default="bfloat16", choices=["bfloat16", "float32"])
    return ap


def describe_model(config) -> str:
    """One line about the model from what its configuration says of itself: the architecture's
    name and every size among its config.json keys (the reference's line, src/arch/llama.rs:74-78,
    without knowing which architecture it is)."""
    d = config.to_dict()
    name = (d.get("architectures") or ["model"])[0]
    sizes = ", ".join(f"{k}={v}" for k, v in d.items() if isinstance(v, int) and not isinstance(v, bool) and not k.endswith("_token_id"))
    return f"{name}: {sizes}"


def parse_ids(text: str) -> List[int]:
    parts = [p for p in re.split(r"[\s,]+", text.strip()) if p]
    try:
        return [int(p) for p in parts]
    except ValueError:
        raise SystemExit(f"Error: the prompt must be token ids (this engine has no tokenizer), got {text!r}")


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    import torch
    from . import Engine, load_config, random_model_tensors, write_model_folder

    if args.command == "init":
        with open(args.config) as f:
            from .config import config_from_dict
            config = config_from_dict(json.load(f))
        dtype = torch.bfloat16 if args.weights_dtype == "bfloat16" else torch.float32
        write_model_folder(args.out, config, random_model_tensors(config, args.seed, dtype=dtype))
        print(f"Wrote {args.out} (seed {args.seed})", file=sys.stderr)
        return 0
    if args.command in ("chat", "serve"):
        print(f"Error: `{args.command}` is not part of this engine (it needs a tokenizer"
              f"{' and an HTTP server' if args.command == 'serve' else ''}); use `complete` with token ids", file=sys.stderr)
        return 1
    if not args.model:
        print("Error: -m/--model is required", file=sys.stderr)
        return 1
    try:
        engine = Engine.from_folder(args.model, dtype=args.dtype, page_size=args.page_size, num_pages=args.num_pages,
                                    max_requests=8, max_batch_tokens=args.max_batch_tokens, log=True)
    except Exception as e:  # configuration, weights or kernels: one line, as the reference's main does
        print(f"Error: {e}", file=sys.stderr)
        return 1
    cfg = engine.config
    print(describe_model(cfg), file=sys.stderr)
    engine.measure_device_time()
    prompt = parse_ids(args.prompt)
    stop = parse_ids(args.stop) if args.stop else list(getattr(cfg, "eos_token_id", ()))
    print(f"Prompt tokens: {len(prompt)}", file=sys.stderr)
    start = time.perf_counter()
    out = engine.generate([prompt], max_new_tokens=args.max_tokens, temperature=args.temperature, top_k=args.top_k,
                          top_p=args.top_p, seed=args.seed, stop_token_ids=stop)[0]
    wall = time.perf_counter() - start
    st = engine.last_stats
    first = max(st.first_token_seconds, 1e-9)
    print(f"Prefill: {len(prompt)} tokens in {first:.2f}s ({len(prompt) / first:.1f} tok/s)", file=sys.stderr)
    print(" ".join(str(t) for t in out))
    rest = max(wall - first, 1e-9)
    gpu = max(st.device_seconds - st.first_token_device_seconds, 0.0)     # the device's share of the decoding time
    print(f"Generated: {len(out)} tokens in {rest:.2f}s ({max(len(out) - 1, 0) / rest:.1f} tok/s)  "
          f"[gpu={gpu:.2f}s overhead={rest - gpu:.2f}s = {(rest - gpu) / rest * 100:.1f}%]", file=sys.stderr)
    from .kernels import kernels
    if kernels().times is not None:       # LLM_PERF: the per-kernel table (src/backend/metal/mod.rs:337-400)
        kernels().times.dump()
    return 0


if __name__ == "__main__":
    sys.exit(main())
