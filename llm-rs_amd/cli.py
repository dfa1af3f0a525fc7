"""Command line in the reference's manner (src/cli/mod.rs:5-69, src/main.rs:84-151):

    llm-rs -m MODEL_DIR complete -p "1 15 27 3" [-n 256] [--temperature 0.7 --top-k 40 --top-p 0.9 --seed 42]
    llm-rs --config config.json --random-weights 0 complete --prompt-len 2048 -n 64
    llm-rs (-m MODEL_DIR | --config FILE --random-weights SEED) replay --out DIR --max-tokens N   < steps.jsonl
    llm-rs (-m MODEL_DIR | --config FILE --random-weights SEED) bench [--prompt-len 2048 --batch 8 --context 2048]
    llm-rs init --config config.json --seed 0 --out MODEL_DIR        (random weights written as a model folder)

`-m/--model` is a folder with config.json and model.safetensors (the reference
takes a GGUF file); `--config FILE --random-weights SEED` makes the weights of that
configuration on the device from the seed instead, without a folder in between (a
70B shape needs no 141 GB of files to be timed).  There is no tokenizer in this
engine, so the prompt is token ids, separated by spaces or commas (or
`--prompt-len N` random ones), and the completion is printed as ids.
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
    ap.add_argument("--config", help="a config.json; with --random-weights in place of --model")
    ap.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                    help="weights drawn from this seed for the configuration of --config (or of --model's folder)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "f32"],
                    type=lambda d: {"bf16": "bfloat16", "f32": "float32", "fp32": "float32"}.get(d, d))
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=None, help="KV pages (default: sized from free memory)")
    ap.add_argument("--max-batch-tokens", type=int, default=2048,
                    help="tokens a step may run (the reference's MAX_TOKENS_PER_STEP); longer prompts are cut into portions")
    sub = ap.add_subparsers(dest="command", required=True)
    c = sub.add_parser("complete", help="Single-shot completion of a prompt given as token ids")
    c.add_argument("-p", "--prompt", "--prompt-ids", dest="prompt", default=None, help="token ids, e.g. \"1 15 27\"")
    c.add_argument("--prompt-len", type=int, default=None, help="in place of --prompt: this many random token ids (drawn from --seed)")
    c.add_argument("-n", "--max-tokens", type=int, default=256)
    c.add_argument("--stop", default="", help="token ids that end the completion (default: eos_token_id of the config)")
    _add_sampling(c)
    ch = sub.add_parser("chat", help="(not available: needs a tokenizer)")
    ch.add_argument("-s", "--system", default=None)
    _add_sampling(ch)
    sv = sub.add_parser("serve", help="(not available: no HTTP server in this engine)")
    sv.add_argument("-p", "--port", type=int, default=8080)
    r = sub.add_parser("replay", help="Feed token ids from standard input through the model step by step and write logits (bin/trace_run)")
    r.add_argument("--out", required=True, help="folder for <step>.f32 files")
    r.add_argument("--max-tokens", type=int, required=True, help="most tokens live requests hold at any time, each rounded up to 64")
    b = sub.add_parser("bench", help="Prompt and decode throughput of this model (examples/bench_throughput.rs)")
    b.add_argument("--prompt-len", type=int, default=2048)
    b.add_argument("--batch", type=int, default=8)
    b.add_argument("--context", type=int, default=2048, help="tokens each decoding request has in the cache")
    b.add_argument("--steps", type=int, default=20)
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


def _random_ids(vocab: int, n: int, seed: int) -> List[int]:
    import torch
    return torch.randint(0, vocab, (max(n, 1),), generator=torch.Generator().manual_seed(seed)).tolist()


def _engine(args, Engine, load_config):
    """The engine the arguments name: a model folder's, or a configuration's with weights from a seed."""
    if args.model is None and args.config is None:
        raise ValueError("-m/--model is required (or --config FILE --random-weights SEED)")
    if args.config is not None and args.random_weights is None:
        raise ValueError("--config gives no weights: add --random-weights SEED, or name a model folder with -m")
    kw = dict(dtype=args.dtype, page_size=args.page_size, num_pages=args.num_pages, max_batch_tokens=args.max_batch_tokens, log=True)
    if args.command == "replay":
        from .engine.trace import TRACE_ROUND_TO
        if TRACE_ROUND_TO % args.page_size:
            raise ValueError(f"--page-size {args.page_size} must divide {TRACE_ROUND_TO}")
        kw.update(num_pages=max(-(-args.max_tokens // args.page_size), 1), max_requests=64)
    elif args.command == "bench":
        need = args.batch * (-(-(args.context + args.steps + 8) // args.page_size)) + -(-args.prompt_len // args.page_size) + 8
        kw.update(max_requests=max(args.batch + 1, 8), num_pages=args.num_pages or need,
                  max_batch_tokens=max(args.max_batch_tokens, args.prompt_len))
    else:
        kw.update(max_requests=8)
    if args.random_weights is None:
        return Engine.from_folder(args.model, **kw)
    if args.config is not None:
        from .config import config_from_dict
        with open(args.config) as f:
            config = config_from_dict(json.load(f))
    else:
        config = load_config(args.model)
    return Engine.from_random(config, args.random_weights, **kw)


def _bench(engine, args) -> int:
    """A prompt of --prompt-len tokens in one step, then --steps decode steps of --batch requests that each hold
    --context tokens, through the engine's own step function; tokens a second of each on standard output as JSON."""
    import torch
    from . import StepEntry
    vocab = engine.model.spec.vocab_size
    positions = engine.max_seq_len
    if args.prompt_len > positions or args.context + args.steps + 4 > positions:
        print(f"Error: the model has {positions} positions", file=sys.stderr)
        return 1

    def timed(fn, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    prompt = _random_ids(vocab, args.prompt_len, 1)
    slot = engine.open_request()
    run_prompt = lambda i: engine.step([StepEntry(slot, 0, prompt, [len(prompt) - 1])])
    run_prompt(0)
    prefill_s = timed(run_prompt, 3)
    engine.close_request(slot)
    slots = [engine.open_request() for _ in range(args.batch)]
    for j, s in enumerate(slots):           # fill the caches, a budget's worth of tokens at a time
        ids = _random_ids(vocab, args.context, 2 + j)
        for at in range(0, args.context, engine.max_batch_tokens):
            engine.step([StepEntry(s, at, ids[at:at + engine.max_batch_tokens], [])])
    decode = lambda i: engine.step([StepEntry(s, args.context + i, [(7 * i + j) % vocab], [0]) for j, s in enumerate(slots)])
    for i in range(4):
        decode(i)
    base = 4
    step_s = timed(lambda i: decode(base + i), args.steps)
    for s in slots:
        engine.close_request(s)
    print(json.dumps({"prefill_tokens": args.prompt_len, "prefill_tok_s": round(args.prompt_len / prefill_s, 1),
                      "prefill_ms": round(prefill_s * 1e3, 3), "decode_batch": args.batch, "decode_context": args.context,
                      "decode_tok_s": round(args.batch / step_s, 1), "decode_ms_per_step": round(step_s * 1e3, 4),
                      "dtype": args.dtype}))
    from .kernels import kernels
    if kernels().times is not None:
        kernels().times.dump()
    return 0


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
    if args.command == "complete" and (args.prompt is None) == (args.prompt_len is None):
        print("Error: complete needs a prompt: -p/--prompt token ids, or --prompt-len N", file=sys.stderr)
        return 1
    try:
        engine = _engine(args, Engine, load_config)
    except Exception as e:  # configuration, weights or kernels: one line, as the reference's main does
        print(f"Error: {e}", file=sys.stderr)
        return 1
    if args.command == "replay":
        from .engine.trace import TraceReplayer, replay_lines
        return replay_lines(TraceReplayer.for_engine(engine), sys.stdin, args.out)
    if args.command == "bench":
        return _bench(engine, args)
    cfg = engine.config
    print(describe_model(cfg), file=sys.stderr)
    engine.measure_device_time()
    if args.prompt is not None:
        prompt = parse_ids(args.prompt)
    else:
        prompt = _random_ids(engine.model.spec.vocab_size, args.prompt_len, args.seed)
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
