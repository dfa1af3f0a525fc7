#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The default run is the Llama-3.1-8B shape with random bfloat16 weights: 8
requests, each with 2,048 tokens of context already in the cache, decode K steps
(one token per request per step, sampled greedily on the device, ids read back),
and report decoded tokens a second.  The same line carries a 2,048-token prefill,
the decode step's share of the HBM roofline, and decode at batch 1 and 64.
A "step" is one decode step.  Counterpart of the reference's timing lines
(src/main.rs:108-112, :141-150) and examples/bench_throughput.rs, in-process.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X, published: HBM3E 8 TB/s; dense MFMA bf16 2.5 PFLOP/s, fp32 157.3 TFLOP/s
PEAK_HBM = 8.0e12
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

LLAMA_8B = dict(
    architectures=["LlamaForCausalLM"], num_hidden_layers=32, hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=8192, rms_norm_eps=1e-5, tie_word_embeddings=False, hidden_act="silu")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048, help="tokens each request has in the cache when decoding starts")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="other decode batch sizes to report")
    ap.add_argument("--only", default="", choices=["", "prefill", "decode"], help="for profiling: time one phase only")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from llm_rs_amd import Engine, LlamaConfig, StepEntry

    full_layers = LLAMA_8B["num_hidden_layers"]
    cfg_dict = dict(LLAMA_8B)
    if args.layers:
        cfg_dict["num_hidden_layers"] = args.layers
    config = LlamaConfig.from_dict(cfg_dict)
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    page_size = 16
    ctx_pages = -(-(args.context + args.steps + args.warmup + 8) // page_size)
    num_pages = max_batch * ctx_pages + 8
    t0 = time.time()
    engine = Engine.from_random(config, seed=0, dtype=args.dtype, device="cuda:0", page_size=page_size,
                                num_pages=num_pages, max_requests=max(max_batch, 8),
                                max_batch_tokens=max(args.prefill_tokens, 2048))
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    vocab = config.vocab_size
    gen = torch.Generator().manual_seed(0)

    def prompt(n):
        return torch.randint(0, vocab, (n,), generator=gen).tolist()

    def timed(fn, reps):
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / reps

    # ---- prefill: one request, its whole prompt in one step, the last logits wanted
    def prefill_once():
        slot = engine.open_request()
        engine.step([StepEntry(slot, 0, toks, [len(toks) - 1])])
        engine.close_request(slot)

    toks = prompt(args.prefill_tokens)
    prefill_once()
    prefill_s = timed(prefill_once, 3 if args.only != "decode" else 1)
    spec = engine.model.spec
    D, F, V, L = config.hidden_size, config.intermediate_size, vocab, config.num_hidden_layers
    Hq, Hkv = config.num_attention_heads * config.head_dim, config.num_key_value_heads * config.head_dim
    T = args.prefill_tokens
    linear = 2 * T * L * (D * (Hq + 2 * Hkv) + Hq * D + 3 * D * F) + 2 * V * D
    attention = L * 2 * 2 * Hq * T * (T + 1) // 2      # QK^T and PV over the causal half
    prefill_flops = linear + attention
    print(f"[bench] prefill {T} tokens: {prefill_s * 1e3:.1f} ms", file=sys.stderr, flush=True)

    # ---- decode
    def decode_run(batch, steps, warmup):
        slots = [engine.open_request() for _ in range(batch)]
        for s in slots:                         # fill each request's cache with `context` tokens
            p, at = prompt(args.context), 0
            while at < len(p):
                n = min(2048, len(p) - at)
                engine.step([StepEntry(s, at, p[at:at + n], [])])
                at += n
        pos = [args.context] * batch
        last = [1] * batch
        state = {"last": last}

        def one_step():
            entries = [StepEntry(s, pos[i], [state["last"][i]], [0]) for i, s in enumerate(slots)]
            logits = engine.step(entries)
            ids = engine.sampler.sample(logits, engine.runner.ctx.sampling, True).cpu().tolist()
            state["last"] = ids
            for i in range(batch):
                pos[i] += 1

        for _ in range(warmup):
            one_step()
        sec = timed(one_step, steps)
        for s in slots:
            engine.close_request(s)
        return sec

    if args.only == "prefill":
        print(json.dumps({"prefill_ms": round(prefill_s * 1e3, 3), "tokens": T}))
        return 0
    step_s = decode_run(args.batch, args.steps, args.warmup)
    print(f"[bench] decode batch {args.batch}: {step_s * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
    point_values = {}
    for b in points:
        s = decode_run(b, max(args.steps // 2, 8), max(args.warmup // 2, 2))
        point_values[f"decode_b{b}"] = round(b / s, 1)
        print(f"[bench] decode batch {b}: {s * 1e3:.3f} ms/step", file=sys.stderr, flush=True)

    weight_bytes = engine.model.weight_bytes_per_step()
    cache_bytes = args.batch * (args.context + args.warmup + args.steps // 2) * engine.cache.bytes_per_token()
    achieved = (weight_bytes + cache_bytes) / step_s
    value = args.batch / step_s
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    line = {
        "metric": f"decode tok/s at batch {args.batch} (8B {short}); prefill tok/s at {T} tokens and batch {'/'.join(str(p) for p in points)} alongside",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic (random weights, uniform random token ids)",
        "config": {"model": "Llama-3.1-8B shape", "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers_run": L, "layers_of_config": full_layers,
                   "hidden_size": D, "num_attention_heads": config.num_attention_heads,
                   "num_key_value_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                   "intermediate_size": F, "vocab_size": V, "max_context": config.max_position_embeddings,
                   "page_size": page_size, "prefill_tokens": T},
        "prefill": {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(prefill_flops / prefill_s / PEAK_FLOPS[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM, 4)},
        "points": point_values,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
