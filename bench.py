#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--workload decode8b|serve1b|mixed70b|sizes|sizes1b|prompts|long|widths|portions]

The default run (`decode8b`) is the Llama-3.1-8B shape with random bfloat16 weights: 8
requests, each with 2,048 tokens of context in the cache, decode K steps through the
engine's own loop (submit / advance: one token per request per step, sampled greedily
on the device, ids read back; the scheduler plans the next step while one is in flight),
and report decoded tokens a second.  The same line carries a 2,048-token prefill,
the decode step's share of the HBM roofline, decode at batch 1 and 64, and the
host's share of a step (wall time minus the device's, from events around the step).
A "step" is one decode step.  Counterpart of the reference's timing lines
(src/main.rs:108-112, :141-150) and examples/bench_throughput.rs, in-process.

The other workloads print one line of the same form each:
  serve1b   Llama-3.2-1B shape, 256 requests at once through submit()/advance(), prompts
            uniform in 128..4096 tokens, 256 new tokens each (continuous batching with
            chunked prefill); value = generated tokens a second; a step is a scheduler step.
  mixed70b  Llama-3.1-70B shape, all 80 layers: 16 requests decoding at context 4096 beside
            one 2,048-token prompt portion, as one step; value = tokens a second of that step.
  sizes     the 8B shape at further sizes: decode at context 8128 (up to the configuration's 8192 positions;
            batch 1/8/64) and at batch 128/256 (context 2048), each with its share of the HBM roofline.
  sizes1b   the 1B shape decoding at batch 1/8/64 (context 2048) with its shares of the HBM roofline: batch 1 is
            the case the reference states its own bandwidth figure for.
  prompts   the 8B shape's prompt step at lengths from 256 to 8192 tokens, among them lengths one token past whole
            tiles: tokens a second and the share of the matrix cores' peak for each; value = the 2,048-token one.
  long      the 8B shape with the 131,072 positions of Llama 3.1: one request decoding over 131,000 keys and four over
            32,700 each, with their shares of the HBM roofline (filling the caches takes about ten seconds).
  widths    the four products of a layer alone, at widths that are none of the three Llama shapes the kernels' choices
            were timed on (hidden 1536 to 6144, odd intermediates), at 1, 8, 64, 256 and 2048 rows: GB/s of weights or
            TFLOP/s for each, so that a width that falls into a poor choice shows; value = the worst share of the best
            share seen at the same number of rows.
  portions  the attention of one request's prompt portion of 2,048 tokens alone (8B shape's heads), over caches of
            2,048 (the whole prompt: causal) to 131,072 keys: TFLOP/s for each; value = the one over 65,536 keys.
With LLM_PERF set in the environment every kernel call is timed by itself and a table
by kernel goes to stderr (the reference's switch, src/backend/metal/mod.rs:235,321-400).
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


def _llama(layers, hidden, heads, kv_heads, head_dim, inter, factor, tied):
    return dict(
        architectures=["LlamaForCausalLM"], num_hidden_layers=layers, hidden_size=hidden, num_attention_heads=heads,
        num_key_value_heads=kv_heads, head_dim=head_dim, intermediate_size=inter, vocab_size=128256, rope_theta=500000.0,
        rope_scaling=dict(rope_type="llama3", factor=factor, low_freq_factor=1.0, high_freq_factor=4.0,
                          original_max_position_embeddings=8192),
        max_position_embeddings=8192, rms_norm_eps=1e-5, tie_word_embeddings=tied, hidden_act="silu")


LLAMA_8B = _llama(32, 4096, 32, 8, 128, 14336, 8.0, False)
LLAMA_1B = _llama(16, 2048, 32, 8, 64, 8192, 32.0, True)
LLAMA_70B = _llama(80, 8192, 64, 8, 128, 28672, 8.0, False)
SHAPES = {"Llama-3.1-8B shape": LLAMA_8B, "Llama-3.2-1B shape": LLAMA_1B, "Llama-3.1-70B shape": LLAMA_70B}
WORKLOADS = ("decode8b", "serve1b", "mixed70b", "sizes", "sizes1b", "prompts", "long", "widths", "portions")


def flat_config(model: str, layers_run: int, global_batch: int, seq_len: int, page_size: int, **more) -> dict:
    """The `config` of a line: every size of the shape by name, flat, at most 20 keys."""
    d = SHAPES[model]
    out = {"model": model, "global_batch": global_batch, "seq_len": seq_len, "parallelism": "single GPU",
           "layers_run": layers_run, "layers_of_config": d["num_hidden_layers"], "hidden_size": d["hidden_size"],
           "num_attention_heads": d["num_attention_heads"], "num_key_value_heads": d["num_key_value_heads"],
           "head_dim": d["head_dim"], "intermediate_size": d["intermediate_size"], "vocab_size": d["vocab_size"],
           "max_context": d["max_position_embeddings"], "page_size": page_size}
    out.update(more)
    assert len(out) <= 20 and all(not isinstance(v, (dict, list)) for v in out.values())
    return out


def base_line(metric: str, value: float, steps: int, warmup: int, step_s: float, dtype: str, config: dict) -> dict:
    return {"metric": metric, "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if dtype == "bfloat16" else "fp32",
            "data": "synthetic (random weights, uniform random token ids)", "config": config}


def roofline(bytes_per_step: float, step_s: float) -> dict:
    achieved = bytes_per_step / step_s
    return {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM, 4)}


def host_share(wall_s: float, device_s: float) -> dict:
    """Wall time of a step against the device's time for it (events before its first kernel and after
    sampling): what is left is the host's (src/main.rs:141-150 prints the same three figures)."""
    return {"wall_ms_per_step": round(wall_s * 1e3, 4), "device_ms_per_step": round(device_s * 1e3, 4),
            "overhead_frac": round(max(wall_s - device_s, 0.0) / wall_s, 4)}


def prefill_flops(d: dict, layers: int, T: int, start: int = 0) -> int:
    """Operations of a portion of T tokens from position `start`: the products of every layer, QK^T and PV
    over the keys each token sees, and the output matrix for one row."""
    D, F, V = d["hidden_size"], d["intermediate_size"], d["vocab_size"]
    Hq, Hkv = d["num_attention_heads"] * d["head_dim"], d["num_key_value_heads"] * d["head_dim"]
    linear = 2 * T * layers * (D * (Hq + 2 * Hkv) + Hq * D + 3 * D * F) + 2 * V * D
    keys_seen = T * start + T * (T + 1) // 2
    return linear + layers * 2 * 2 * Hq * keys_seen


def decode_line(args, layers, step_s, weight_bytes, cache_bytes_per_token, prefill_s, points, host) -> dict:
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    T = args.prefill_tokens
    line = base_line(
        f"decode tok/s at batch {args.batch} (8B {short}); prefill tok/s at {T} tokens"
        + (f" and batch {'/'.join(p.split('_b')[1] for p in points if '_ctx' not in p and p != 'decode_b256')}" if points else "") + " alongside",
        args.batch / step_s, args.steps, args.warmup, step_s, args.dtype,
        flat_config("Llama-3.1-8B shape", layers, args.batch, args.context, 16, prefill_tokens=T))
    line["prefill"] = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
                       "frac": round(prefill_flops(LLAMA_8B, layers, T) / prefill_s / PEAK_FLOPS[args.dtype], 4)}
    cache_bytes = args.batch * (args.context + args.warmup + args.steps // 2) * cache_bytes_per_token
    line["roofline"] = roofline(weight_bytes + cache_bytes, step_s)
    line["points"] = points
    line["host"] = host
    return line


def serve_line(args, layers, n_requests, prompt_tokens, generated, seconds, steps, device_s, preemptions, budget) -> dict:
    line = base_line(
        f"generated tok/s, {n_requests} requests at once, prompts uniform in 128..4096, {args.new_tokens} new tokens each "
        f"(1B bf16, continuous batching with chunked prefill)",
        generated / seconds, steps, 0, seconds / max(steps, 1), args.dtype,
        flat_config("Llama-3.2-1B shape", layers, n_requests, 4096 + args.new_tokens, 16,
                    max_batch_tokens=budget, new_tokens=args.new_tokens))
    line["total_tokens_per_s"] = round((prompt_tokens + generated) / seconds, 1)
    line["prompt_tokens"] = prompt_tokens
    line["generated_tokens"] = generated
    line["seconds"] = round(seconds, 3)
    line["preemptions"] = preemptions
    line["host"] = host_share(seconds / max(steps, 1), device_s / max(steps, 1))
    return line


def mixed_line(args, layers, step_s, weight_bytes, cache_bytes, host) -> dict:
    n_dec, chunk, ctx = 16, 2048, 4096
    tokens = n_dec + chunk
    line = base_line(
        f"tokens/s of one step: {n_dec} requests decoding at context {ctx} beside a {chunk}-token prompt portion (70B bf16)",
        tokens / step_s, args.steps, args.warmup, step_s, args.dtype,
        flat_config("Llama-3.1-70B shape", layers, n_dec + 1, ctx, 16, decodes=n_dec, prefill_chunk=chunk))
    flops = prefill_flops(LLAMA_70B, layers, chunk, start=ctx - chunk) + \
        n_dec * (prefill_flops(LLAMA_70B, layers, 1, start=ctx - 1) - 2 * 128256 * 8192) + n_dec * 2 * 128256 * 8192
    line["compute"] = {"bound": "mfma", "achieved": round(flops / step_s / 1e12, 1), "peak": PEAK_FLOPS[args.dtype] / 1e12,
                       "unit": "TFLOP/s", "frac": round(flops / step_s / PEAK_FLOPS[args.dtype], 4)}
    line["roofline"] = roofline(weight_bytes + cache_bytes, step_s)
    line["host"] = host
    return line


def sizes_line(args, layers, points, fractions, first_step_s=0.0, model="Llama-3.1-8B shape") -> dict:
    """`value` and `ms_per_step` are the first point's; the others stand under `points`."""
    first = next(iter(points))
    what = ("further sizes (context 8128; batch 128 and 256)" if model == "Llama-3.1-8B shape"
            else "batch 1, 8 and 64 (context 2048; batch 1 is the reference's own headline case)")
    line = base_line(f"decode tok/s of the {model.split()[0].split('-')[-1]} shape at {what}, each with its share of the HBM roofline",
                     points[first], args.steps, args.warmup, first_step_s, args.dtype,
                     flat_config(model, layers, 0, 8192 if model == "Llama-3.1-8B shape" else 2048, 16))
    line["points"] = points
    line["roofline_frac"] = fractions
    return line


def long_line(args, layers, points, fractions, first_step_s=0.0) -> dict:
    """`value` and `ms_per_step` are the first point's (one request over the longest cache)."""
    first = next(iter(points))
    line = base_line("decode tok/s of the 8B shape over long caches (131,072 positions), each with its share of the HBM roofline",
                     points[first], args.steps, args.warmup, first_step_s, args.dtype,
                     flat_config("Llama-3.1-8B shape", layers, 0, 131072, 16, max_context=131072))
    line["points"] = points
    line["roofline_frac"] = fractions
    return line


def prompts_line(args, layers, points, fractions, first_step_s=0.0) -> dict:
    """`value` and `ms_per_step` are the 2,048-token prompt's (the first point); a step is one prompt step."""
    first = next(iter(points))
    line = base_line("prefill tok/s of the 8B shape over prompt lengths (one request, its whole prompt in one step), each with its "
                     "share of the matrix cores' peak", points[first], args.steps, args.warmup, first_step_s, args.dtype,
                     flat_config("Llama-3.1-8B shape", layers, 1, 8192, 16))
    line["points"] = points
    line["peak_frac"] = fractions
    return line


# ---- measurements (need the GPU) -------------------------------------------------------------------------------

class Bench:
    def __init__(self, args, shape: dict, num_pages: int, max_requests: int, max_batch_tokens: int):
        import torch
        from llm_rs_amd import Engine, LlamaConfig
        self.torch = torch
        d = dict(shape)
        if args.layers:
            d["num_hidden_layers"] = args.layers
        self.config = LlamaConfig.from_dict(d)
        t0 = time.time()
        self.engine = Engine.from_random(self.config, seed=0, dtype=args.dtype, device="cuda:0", page_size=16,
                                         num_pages=num_pages, max_requests=max_requests, max_batch_tokens=max_batch_tokens)
        self.max_batch_tokens = max_batch_tokens
        torch.cuda.synchronize()
        print(f"[bench] model ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
        self.gen = torch.Generator().manual_seed(0)

    def prompt(self, n):
        return self.torch.randint(0, self.config.vocab_size, (n,), generator=self.gen).tolist()

    def timed(self, fn, reps):
        self.torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(reps):
            fn()
        self.torch.cuda.synchronize()
        return (time.perf_counter() - t) / reps

    def fill(self, slot, tokens, chunk=2048):
        from llm_rs_amd import StepEntry
        at = 0
        while at < len(tokens):
            n = min(chunk, len(tokens) - at)
            self.engine.step([StepEntry(slot, at, tokens[at:at + n], [])])
            at += n

    def device_seconds(self, fn, reps):
        """Device time of `fn` (a step and its sampling), from an event before the step's first kernel to one after."""
        torch, runner = self.torch, self.engine.runner
        runner.time_device = True
        pairs = []
        for _ in range(reps):
            fn()
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            pairs.append((runner.started, end))
        runner.time_device = False
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in pairs) * 1e-3 / reps

    def decode_run(self, batch, context, steps, warmup, with_device_time=False):
        """Seconds per decode step of `batch` requests over `context` keys each, through the engine's own loop
        (submit / advance: the scheduler, one step in flight while the next is planned), and the device's share."""
        engine = self.engine
        measured = min(steps, 16) if with_device_time else 0
        # a request's portion of a step is capped so that the `batch` prompts, all of one length, run side by side
        # and end in the same step: the requests then decode over equal contexts
        engine.cache.core.set_max_chunk(max(1, self.max_batch_tokens // batch))
        requests = [engine.submit(self.prompt(context), max_new_tokens=warmup + steps + measured + 4) for _ in range(batch)]
        for _ in range(context * batch + 8):        # the prompts, in equal portions side by side: they end in the same step
            if len(engine.advance()) == batch:
                break
        else:
            raise RuntimeError("the requests did not come to decode together")

        def one_step():
            if len(engine.advance()) != batch:
                raise RuntimeError("a decode step did not give every request a token")

        for _ in range(warmup):
            one_step()
        sec = self.timed(one_step, steps)
        dev = self.device_seconds(one_step, measured) if with_device_time else None
        for r in requests:
            engine.cancel(r)
        while engine.has_unfinished():              # (the step in flight lands; what it sampled is nobody's)
            engine.advance()
        engine.cache.core.set_max_chunk(0)
        return sec, dev


def run_decode8b(args) -> dict:
    from llm_rs_amd import StepEntry
    # further points: "batch" (at --context) or "batch@context"
    points = [(int(p.split("@")[0]), int(p.split("@")[1]) if "@" in p else args.context) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + [bt for bt, _ in points])
    pages_for = lambda bt, ctx: bt * (-(-(ctx + args.steps + args.warmup + 24) // 16))
    b = Bench(args, LLAMA_8B, max([pages_for(args.batch, args.context)] + [pages_for(bt, ctx) for bt, ctx in points]) + 8,
              max(max_batch, 8), max(args.prefill_tokens, 2048))
    engine = b.engine
    toks = b.prompt(args.prefill_tokens)

    def prefill_once():     # one request, its whole prompt in one step, the last logits wanted
        slot = engine.open_request()
        engine.step([StepEntry(slot, 0, toks, [len(toks) - 1])])
        engine.close_request(slot)

    prefill_once()
    prefill_s = b.timed(prefill_once, 3 if args.only != "decode" else 1)
    print(f"[bench] prefill {args.prefill_tokens} tokens: {prefill_s * 1e3:.1f} ms", file=sys.stderr, flush=True)
    if args.only == "prefill":
        return {"prefill_ms": round(prefill_s * 1e3, 3), "tokens": args.prefill_tokens}
    step_s, dev_s = b.decode_run(args.batch, args.context, args.steps, args.warmup, with_device_time=True)
    print(f"[bench] decode batch {args.batch}: {step_s * 1e3:.3f} ms/step (device {dev_s * 1e3:.3f})", file=sys.stderr, flush=True)
    point_values, point_fracs = {}, {}
    weight_bytes, per_token = engine.model.weight_bytes_per_step(), engine.cache.bytes_per_token()
    for bt, ctx in points:
        steps, warmup = max(args.steps // 2, 8), max(args.warmup // 2, 2)
        s, _ = b.decode_run(bt, ctx, steps, warmup)
        key = f"decode_b{bt}" + (f"_ctx{ctx}" if ctx != args.context else "")
        point_values[key] = round(bt / s, 1)
        point_fracs[key] = round((weight_bytes + bt * (ctx + warmup + steps // 2) * per_token) / s / PEAK_HBM, 4)
        print(f"[bench] decode batch {bt} at context {ctx}: {s * 1e3:.3f} ms/step, {point_fracs[key] * 100:.1f}% of the HBM roofline",
              file=sys.stderr, flush=True)
    line = decode_line(args, b.config.num_hidden_layers, step_s, weight_bytes, per_token, prefill_s, point_values, host_share(step_s, dev_s))
    line["points_frac"] = point_fracs
    return line


def run_sizes(args) -> dict:
    steps, warmup = max(args.steps // 2, 8), max(args.warmup // 2, 2)
    long = 8192 - 64        # decoding ends just under the configuration's 8192 positions (block tables 512 pages wide)
    assert steps + warmup <= 56
    small = args.workload == "sizes1b"
    cases = [(1, 2048), (8, 2048), (64, 2048)] if small else [(1, long), (8, long), (64, long), (128, 2048), (256, 2048)]
    pages = max(bt * (-(-(ctx + steps + warmup + 24) // 16)) for bt, ctx in cases) + 8
    b = Bench(args, LLAMA_1B if small else LLAMA_8B, pages, 256, 2048)
    weight_bytes, per_token = b.engine.model.weight_bytes_per_step(), b.engine.cache.bytes_per_token()
    points, fractions, first_s = {}, {}, None
    for batch, ctx in cases:
        s, _ = b.decode_run(batch, ctx, steps, warmup)
        first_s = s if first_s is None else first_s
        key = f"decode_b{batch}_ctx{ctx}"
        points[key] = round(batch / s, 1)
        fractions[key] = round((weight_bytes + batch * (ctx + warmup + steps // 2) * per_token) / s / PEAK_HBM, 4)
        print(f"[bench] {key}: {s * 1e3:.3f} ms/step, {fractions[key] * 100:.1f}% of the HBM roofline", file=sys.stderr, flush=True)
    return sizes_line(args, b.config.num_hidden_layers, points, fractions, first_s,
                      "Llama-3.2-1B shape" if small else "Llama-3.1-8B shape")


def run_long(args) -> dict:
    steps, warmup = 16, 4
    shape = dict(LLAMA_8B, max_position_embeddings=131072)
    cases = [(1, 131072 - 64), (4, 32768 - 64)]
    pages = max(bt * (-(-(ctx + steps + warmup + 24) // 16)) for bt, ctx in cases) + 8
    b = Bench(args, shape, pages, 8, 2048)
    weight_bytes, per_token = b.engine.model.weight_bytes_per_step(), b.engine.cache.bytes_per_token()
    points, fractions, first_s = {}, {}, None
    for batch, ctx in cases:
        t0 = time.time()
        s, _ = b.decode_run(batch, ctx, steps, warmup)
        first_s = s if first_s is None else first_s
        key = f"decode_b{batch}_ctx{ctx}"
        points[key] = round(batch / s, 1)
        fractions[key] = round((weight_bytes + batch * (ctx + warmup + steps // 2) * per_token) / s / PEAK_HBM, 4)
        print(f"[bench] {key}: {s * 1e3:.3f} ms/step, {fractions[key] * 100:.1f}% of the HBM roofline (with filling the caches: "
              f"{time.time() - t0:.1f} s)", file=sys.stderr, flush=True)
    args.steps, args.warmup = steps, warmup
    return long_line(args, b.config.num_hidden_layers, points, fractions, first_s)


def run_prompts(args) -> dict:
    from llm_rs_amd import StepEntry
    lengths = (2048, 256, 512, 1024, 1025, 2049, 4096, 8192)
    b = Bench(args, LLAMA_8B, max(lengths) // 16 + 16, 8, max(lengths))
    engine = b.engine
    reps = max(2, min(args.steps // 8, 8))
    points, fractions, first_s = {}, {}, None
    for T in lengths:
        toks = b.prompt(T)

        def prompt_once():
            slot = engine.open_request()
            engine.step([StepEntry(slot, 0, toks, [T - 1])])
            engine.close_request(slot)

        prompt_once()
        s = b.timed(prompt_once, reps)
        first_s = s if first_s is None else first_s
        points[f"prefill_{T}"] = round(T / s, 1)
        fractions[f"prefill_{T}"] = round(prefill_flops(LLAMA_8B, b.config.num_hidden_layers, T) / s / PEAK_FLOPS[args.dtype], 4)
        print(f"[bench] prompt of {T} tokens: {s * 1e3:.2f} ms, {fractions[f'prefill_{T}'] * 100:.1f}% of the peak", file=sys.stderr, flush=True)
    return prompts_line(args, b.config.num_hidden_layers, points, fractions, first_s)


def run_serve1b(args) -> dict:
    n, new = args.requests, args.new_tokens
    b = Bench(args, LLAMA_1B, (n * (4096 + new)) // 16 + 64, n, args.max_batch_tokens)
    engine, torch = b.engine, b.torch
    lens = torch.randint(128, 4097, (n,), generator=b.gen).tolist()
    prompts = [b.prompt(k) for k in lens]
    engine.generate([prompts[0][:300], prompts[1][:40]], max_new_tokens=4)       # buffers grow, nothing is timed yet
    engine.measure_device_time()
    t0 = time.perf_counter()
    out = engine.generate(prompts, max_new_tokens=new)
    seconds = time.perf_counter() - t0
    st = engine.last_stats
    generated = sum(len(o) for o in out)
    assert all(len(o) == new for o in out)
    print(f"[bench] {n} requests: {st.prompt_tokens} prompt + {generated} generated tokens in {seconds:.2f}s, {st.steps} steps, "
          f"graph replays {engine.runner.graph_replays}", file=sys.stderr, flush=True)
    return serve_line(args, b.config.num_hidden_layers, n, st.prompt_tokens, generated, seconds, st.steps, st.device_seconds,
                      st.preemptions, args.max_batch_tokens)


def run_mixed70b(args) -> dict:
    from llm_rs_amd import StepEntry
    n_dec, chunk, ctx = 16, 2048, 4096
    b = Bench(args, LLAMA_70B, (n_dec + 1) * (ctx // 16 + 2) + 8, 24, 4096)
    engine = b.engine
    dec = [engine.open_request() for _ in range(n_dec)]
    for s in dec:
        b.fill(s, b.prompt(ctx - 1))
    pre = engine.open_request()
    ptoks = b.prompt(ctx)
    b.fill(pre, ptoks[:ctx - chunk])
    last = b.prompt(n_dec)

    def step():     # positions are not advanced: the same step again writes the same cache slots
        logits = engine.step([StepEntry(s, ctx - 1, [last[i]], [0]) for i, s in enumerate(dec)] +
                             [StepEntry(pre, ctx - chunk, ptoks[ctx - chunk:], [chunk - 1])])
        engine.sampler.sample(logits, engine.runner.ctx.sampling, True).cpu()

    for _ in range(max(args.warmup, 1)):
        step()
    step_s = b.timed(step, args.steps)
    dev_s = b.device_seconds(step, min(args.steps, 4))
    print(f"[bench] mixed step: {step_s * 1e3:.2f} ms (device {dev_s * 1e3:.2f})", file=sys.stderr, flush=True)
    cache_bytes = (n_dec * ctx + ctx) * engine.cache.bytes_per_token()
    return mixed_line(args, b.config.num_hidden_layers, step_s, engine.model.weight_bytes_per_step(), cache_bytes,
                      host_share(step_s, dev_s))


def run_widths(args) -> dict:
    """The products q/k/v, o, gate/up and down of one layer at other widths, in a HIP graph, back to back over
    different weights (so that no weight is read twice in a row)."""
    import torch
    from llm_rs_amd.kernels import EPI_ACCUM_F32, EPI_STORE, EPI_SWIGLU, kernels
    k, dev = kernels(), "cuda:0"
    # (hidden, heads x head size of q, kv heads x head size, intermediate)
    shapes = [(1536, 1536, 256, 8960), (2560, 2560, 640, 6912), (3072, 3072, 1024, 8192), (3584, 3584, 512, 18944),
              (5120, 5120, 1024, 13824), (6144, 6144, 1024, 16384), (4096, 4096, 1024, 11008)]
    rows_list = (1, 8, 64, 256, 2048)
    points, best = {}, {}
    for hidden, qd, kvd, inter in shapes:
        products = {"qkv": (qd + 2 * kvd, hidden, EPI_STORE), "o": (hidden, qd, EPI_ACCUM_F32),
                    "gate_up": (2 * inter, hidden, EPI_SWIGLU), "down": (hidden, inter, EPI_ACCUM_F32)}
        for name, (N, K, epi) in products.items():
            copies = max(2, min(8, int(600e6 // (N * K * 2))))          # enough different weights to pass the caches
            ws = [(torch.randn(N, K, device=dev) * 0.02).bfloat16() for _ in range(copies)]
            for M in rows_list:
                x = torch.randn(M, K, device=dev).bfloat16()
                out = torch.zeros(M, N // 2 if epi == EPI_SWIGLU else N, device=dev,
                                  dtype=torch.float32 if epi == EPI_ACCUM_F32 else torch.bfloat16)
                n_ws = k.gemm_workspace_floats(M, N, K)
                wsp = torch.empty(max(n_ws, 1), dtype=torch.float32, device=dev) if n_ws else None
                for w in ws:
                    k.gemm(x, w, out, epi, wsp)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for _ in range(4):
                        for w in ws:
                            k.gemm(x, w, out, epi, wsp)
                graph.replay()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(5):
                    graph.replay()
                torch.cuda.synchronize()
                sec = (time.perf_counter() - t0) / (5 * 4 * copies)
                hbm = N * K * 2 / sec / PEAK_HBM
                mfma = 2.0 * M * N * K / sec / PEAK_FLOPS["bfloat16"]
                share = max(hbm, mfma)              # of whichever roof the product is nearer to
                key = f"{name}_{N}x{K}_m{M}"
                points[key] = round(share, 4)
                best[M] = max(best.get(M, 0.0), share)
                print(f"[bench] {key}: {sec * 1e6:8.1f} us  {hbm * 100:5.1f}% of HBM  {mfma * 100:5.1f}% of the matrix peak", file=sys.stderr, flush=True)
                del graph
            del ws
    worst = min(points, key=lambda kk: points[kk] / best[int(kk.rsplit("_m", 1)[1])])
    rel = points[worst] / best[int(worst.rsplit("_m", 1)[1])]
    line = base_line("the worst product's share of its roof (HBM for few rows, matrix cores for many) against the best seen at the same "
                     "number of rows, over the four products of a layer at seven other widths", rel, 20, 0, 0.0, "bfloat16",
                     {"model": "other widths", "global_batch": 0, "seq_len": 0, "parallelism": "single GPU"})
    line["unit"] = "ratio"
    line["worst"] = worst
    line["best_share_by_rows"] = {str(m): round(v, 4) for m, v in best.items()}
    line["points"] = points
    return line


def run_portions(args) -> dict:
    """The attention kernel for entries with several tokens, by itself: a portion of 2,048 tokens of one request whose
    cache holds `keys` keys (the portion's own among them), heads and head size of the 8B shape, pages in order."""
    import torch
    from llm_rs_amd.kernels import kernels
    k, dev = kernels(), "cuda:0"
    H, KV, HD, PS, T = LLAMA_8B["num_attention_heads"], LLAMA_8B["num_key_value_heads"], LLAMA_8B["head_dim"], 16, 2048
    points, fractions, first_s = {}, {}, 0.0
    for keys in (2048, 8192, 16384, 32768, 65536, 131072):
        pages = keys // PS
        kc = torch.randn(pages * KV * PS * HD, device=dev).to(torch.bfloat16)
        vc = torch.randn(pages * KV * PS * HD, device=dev).to(torch.bfloat16)
        q = torch.randn(T, H * HD, device=dev).to(torch.bfloat16)
        out = torch.empty_like(q)
        table = torch.arange(pages, dtype=torch.int32, device=dev).reshape(1, pages)
        entry = torch.zeros(T, dtype=torch.int32, device=dev)
        positions = torch.arange(keys - T, keys, dtype=torch.int32, device=dev)
        q_starts = torch.tensor([0, T], dtype=torch.int32, device=dev)
        seq_lens = torch.tensor([keys], dtype=torch.int32, device=dev)

        def call():
            k.attention(q, out, kc, vc, table, entry, positions, q_starts, seq_lens, H, KV, HD, PS, pages, 0, HD ** -0.5, None, keys, 0)

        for _ in range(2 if points else 20):            # (the first calls of the process also see the clocks rise)
            call()
        torch.cuda.synchronize()
        reps = 5
        t0 = time.perf_counter()
        for _ in range(reps):
            call()
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t0) / reps
        flops = 4.0 * H * HD * (T * keys - T * (T - 1) / 2)           # two products, each query over the keys it may see
        if keys == 65536:
            first_s = sec
        points[f"attention_{keys}"] = round(flops / sec / 1e12, 1)
        fractions[f"attention_{keys}"] = round(flops / sec / PEAK_FLOPS["bfloat16"], 4)
        print(f"[bench] portion of {T} tokens over {keys} keys: {sec * 1e6:9.1f} us  {flops / sec / 1e12:6.0f} TFLOP/s", file=sys.stderr, flush=True)
        del kc, vc
    first = "attention_65536"
    line = base_line("TFLOP/s of the attention of a 2,048-token prompt portion alone (8B shape's heads) over caches of 2,048 to 131,072 keys; "
                     "value: over 65,536", points[first], reps, 2, first_s, "bfloat16",
                     {"model": "Llama-3.1-8B shape (attention only)", "global_batch": 1, "seq_len": 65536, "parallelism": "single GPU",
                      "num_attention_heads": H, "num_key_value_heads": KV, "head_dim": HD, "page_size": PS, "portion_tokens": T})
    line["unit"] = "TFLOP/s"
    line["points"] = points
    line["peak_frac"] = fractions
    return line


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 64; 8 for mixed70b)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 8; 2 for mixed70b)")
    ap.add_argument("--workload", default="decode8b", choices=WORKLOADS)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048, help="tokens each request has in the cache when decoding starts")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64,256,1@8128,64@8128",
                    help="other decode points to report (decode8b): batch sizes at --context, or batch@context")
    ap.add_argument("--only", default="", choices=["", "prefill", "decode"], help="for profiling: time one phase only (decode8b)")
    ap.add_argument("--requests", type=int, default=256, help="serve1b: requests submitted at once")
    ap.add_argument("--new-tokens", type=int, default=256, help="serve1b: tokens generated for each request")
    ap.add_argument("--max-batch-tokens", type=int, default=2048, help="serve1b: tokens a scheduler step may run")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    heavy = args.workload == "mixed70b"
    args.steps = args.steps if args.steps is not None else (8 if heavy else 64)
    args.warmup = args.warmup if args.warmup is not None else (2 if heavy else 8)
    line = {"decode8b": run_decode8b, "serve1b": run_serve1b, "mixed70b": run_mixed70b, "sizes": run_sizes, "sizes1b": run_sizes,
            "prompts": run_prompts, "long": run_long, "widths": run_widths, "portions": run_portions}[args.workload](args)
    from llm_rs_amd.kernels import kernels
    if kernels().times is not None:         # LLM_PERF: what was still to be shown of the per-kernel table
        kernels().times.dump()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
