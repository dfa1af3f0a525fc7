"""Each part alone against the plain function of its formula, and the generality
of how parts are put together: a sliding-window attention, a schedule that runs
a layer twice and lets a run read another run's cache, and a toy mixer with
state of its own, a feed-forward that routes each token to one of several experts
and a position encoding that is no rotation, all defined and registered here, in the
test, and built and stepped without a change to the package."""
import math
from types import SimpleNamespace

import pytest
import torch

from llm_rs_amd import (Engine, ExtraPart, FixedState, LayerSpec, ModelSpec, PartSpec, RunSpec, StepEntry, StepRunner,
                        register_architecture)
from llm_rs_amd.cache import CacheManager, PagedKV
from llm_rs_amd.parts import (Block, FeedForward, Mixer, PositionEncoding, TensorSpec, build_block, build_feed_forward,
                              build_mixer, build_norm, build_position, register_block, register_feed_forward, register_mixer,
                              register_position)
from plain_llama import plain_attention, plain_inv_freq, plain_rmsnorm, plain_rope, plain_swiglu

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 2e-5, torch.bfloat16: 1.5e-2}


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


class Harness:
    """Runs `fn(ctx, cache_views)` as a step's model, over a real cache manager and step function."""

    def __init__(self, needs, dtype, page_size=16, num_pages=64):
        self.cache = CacheManager(needs, dtype, DEV, page_size, num_pages, max_requests=8)
        self.stub = SimpleNamespace(spec=SimpleNamespace(vocab_size=1 << 30, max_positions=1 << 20), forward=None)
        self.runner = StepRunner(self.stub, self.cache, DEV)

    def run(self, entries, fn):
        self.stub.forward = fn
        return self.runner.run(entries)


def close(got, ref, dtype):
    scale = max(float(ref.abs().max()), 1.0)
    return float((got.double().cpu() - ref).abs().max()) <= TOL[dtype] * scale


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    norm = build_norm(PartSpec("rmsnorm", "n", {"size": 72, "eps": 1e-3}), dtype)
    assert norm.tensors() == {"n.weight": TensorSpec((72,), "norm")}
    w = rnd((72,), 0) * 0.1 + 1
    norm.load({"n.weight": w.bfloat16()}, DEV)
    assert norm.weight.dtype == torch.float32
    h = rnd((5, 72), 1, 2.0).to(DEV)
    out = torch.empty((5, 72), dtype=dtype, device=DEV)
    norm.forward(None, h, out)
    assert close(out, plain_rmsnorm(h.double().cpu(), w.bfloat16().double(), 1e-3), dtype)


def test_rotary_part_makes_the_table():
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    rope = build_position({"kind": "rope", "head_dim": 48, "rotary_dim": 32, "theta": 500000.0, "layout": "interleaved", "scaling": sc}, torch.float32)
    table, rotary_dim, interleaved = rope.rotary()
    assert rotary_dim == 32 and interleaved and torch.equal(table, plain_inv_freq(32, 500000.0, sc))
    assert build_position(None, torch.float32) is None
    with pytest.raises(KeyError, match="unknown position encoding"):
        build_position({"kind": "alibi"}, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_part(dtype):
    ffn = build_feed_forward(PartSpec("swiglu", "f", {"hidden_size": 40, "intermediate_size": 88}), dtype)
    ws = {"f.gate_proj.weight": rnd((88, 40), 2, 0.2).bfloat16(), "f.up_proj.weight": rnd((88, 40), 3, 0.2).bfloat16(),
          "f.down_proj.weight": rnd((40, 88), 4, 0.2).bfloat16()}
    assert {n: t.shape for n, t in ffn.tensors().items()} == {n: tuple(t.shape) for n, t in ws.items()}
    ffn.load(ws, DEV)
    x = rnd((7, 40), 5).to(dtype)
    h0 = rnd((7, 40), 6)
    hz = Harness([], dtype)
    out = {}

    def fn(ctx, views):
        h = h0.to(DEV).clone()
        ffn.forward(ctx, x.to(DEV), h)
        out["h"] = h
    s = hz.cache.core.acquire_slot()
    hz.run([StepEntry(s, 0, [0] * 7, [])], fn)
    ref = h0.double() + plain_swiglu(x.double(), *(ws[k].double() for k in ("f.gate_proj.weight", "f.up_proj.weight", "f.down_proj.weight")))
    assert close(out["h"], ref, dtype)


def attention_reference(ws, prefix, x, heads, kv, hd, rope, window, scale=None):
    T = x.shape[0]
    q = (x @ ws[f"{prefix}.q_proj.weight"].double().T).view(T, heads, hd)
    k = (x @ ws[f"{prefix}.k_proj.weight"].double().T).view(T, kv, hd)
    v = (x @ ws[f"{prefix}.v_proj.weight"].double().T).view(T, kv, hd)
    if rope is not None:
        inv = plain_inv_freq(rope["rotary_dim"], rope["theta"], rope.get("scaling"))
        pos = torch.arange(T)
        q, k = plain_rope(q, pos, inv, rope["layout"]), plain_rope(k, pos, inv, rope["layout"])
    o = plain_attention(q, k, v, scale, window).reshape(T, heads * hd)
    return o @ ws[f"{prefix}.o_proj.weight"].double().T


ATTN_CASES = [
    dict(hidden=40, heads=4, kv=2, hd=16, window=None, rotary=16, layout="split_half", ps=4),
    dict(hidden=72, heads=6, kv=2, hd=32, window=None, rotary=32, layout="split_half", ps=16),
    dict(hidden=64, heads=4, kv=4, hd=32, window=9, rotary=16, layout="interleaved", ps=16),      # a window, part of the head rotated
    dict(hidden=48, heads=2, kv=1, hd=64, window=20, rotary=0, layout="split_half", ps=16),        # no position encoding at all
    dict(hidden=56, heads=3, kv=3, hd=48, window=None, rotary=48, layout="split_half", ps=8),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention_part(dtype, case):
    c = SimpleNamespace(**case)
    rope = None if c.rotary == 0 else {"kind": "rope", "head_dim": c.hd, "rotary_dim": c.rotary, "theta": 10000.0, "layout": c.layout}
    att = build_mixer(PartSpec("attention", "a", {"hidden_size": c.hidden, "num_heads": c.heads, "num_kv_heads": c.kv,
                                                  "head_dim": c.hd, "window": c.window, "position": rope}), dtype)
    assert att.cache_need() == PagedKV(c.kv, c.hd, c.window or 0)
    ws = {n: rnd(s.shape, i, 0.15).bfloat16() for i, (n, s) in enumerate(att.tensors().items())}
    att.load(ws, DEV)
    T = 45
    x = rnd((T, c.hidden), 9).to(dtype)
    ref = attention_reference(ws, "a", x.double(), c.heads, c.kv, c.hd, rope, c.window or 0)
    hz = Harness([(att.cache_need(), None)], dtype, page_size=c.ps)
    s = hz.cache.core.acquire_slot()
    got, pos = [], 0
    for n in (7, 2, 16, 1, 1, 11, 1, 6):           # portions and single tokens from the same cache
        def fn(ctx, views, lo=pos, n=n):
            h = torch.zeros((n, c.hidden), dtype=torch.float32, device=DEV)
            att.forward(ctx, x[lo:lo + n].to(DEV), h, views[0])
            got.append(h)
        hz.run([StepEntry(s, pos, [0] * n, [])], fn)
        pos += n
    assert close(torch.cat(got), ref, dtype)
    if c.window:
        assert hz.cache.core.pages_held(s) < -(-T // c.ps) or c.window + c.ps >= T, "pages behind the window go back to the pool"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_alone(dtype):
    H, F = 48, 80
    layer = LayerSpec("prenorm",
                      PartSpec("attention", "b.att", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 1, "head_dim": 32, "window": None,
                                                      "position": {"kind": "rope", "head_dim": 32, "rotary_dim": 32, "theta": 1e4, "layout": "split_half"}}),
                      PartSpec("swiglu", "b.mlp", {"hidden_size": H, "intermediate_size": F}),
                      PartSpec("rmsnorm", "b.n1", {"size": H, "eps": 1e-5}), PartSpec("rmsnorm", "b.n2", {"size": H, "eps": 1e-6}))
    block = build_block(layer, dtype)
    ws = {}
    for i, part in enumerate(block.parts()):
        for n, s in part.tensors().items():
            ws[n] = ((rnd(s.shape, 20 + len(ws)) * 0.1 + 1) if s.kind == "norm" else rnd(s.shape, 20 + len(ws), 0.15)).bfloat16()
        part.load(ws, DEV)
    T = 19
    h0 = rnd((T, H), 3)
    x = h0.double()
    xn = plain_rmsnorm(x, ws["b.n1.weight"].double(), 1e-5)
    x = x + attention_reference(ws, "b.att", xn, 3, 1, 32, layer.mixer.params["position"], 0)
    xn = plain_rmsnorm(x, ws["b.n2.weight"].double(), 1e-6)
    ref = x + plain_swiglu(xn, ws["b.mlp.gate_proj.weight"].double(), ws["b.mlp.up_proj.weight"].double(), ws["b.mlp.down_proj.weight"].double())
    hz = Harness([(block.mixer.cache_need(), None)], dtype)
    s = hz.cache.core.acquire_slot()
    out = {}

    def fn(ctx, views):
        h = h0.to(DEV).clone()
        block.forward(ctx, h, views[0])
        out["h"] = h
    hz.run([StepEntry(s, 0, [0] * T, [])], fn)
    assert close(out["h"], ref, dtype)


# ---- a toy mixer with state of its own, defined here -------------------------------------------

class DecayMixer(Mixer):
    """s_t = decay * s_{t-1} + x_t per request; y_t = s_t W^T.  Its state is one vector per
    request, kept in the request's slot; it needs no pages."""

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden, self.decay = spec.params["hidden_size"], spec.params["decay"]
        self.w = None

    def tensors(self):
        return {self.name("w"): TensorSpec((self.hidden, self.hidden))}

    def load(self, tensors, device):
        self.w = tensors[self.name("w")].to(device=device, dtype=torch.float32)

    def cache_need(self):
        return FixedState((self.hidden,), torch.float32)

    def forward(self, ctx, x, h, cache):
        at = 0
        for slot, start, count in ctx.entries:       # the step's host-side view: (slot, start, count)
            s = cache.state[slot]
            for t in range(at, at + count):
                s.mul_(self.decay).add_(x[t].float())
                h[t] += s @ self.w.T
            at += count


class ToyConfig:
    """Four runs over three layers: decay mixer, attention, the decay layer again (with a state
    of its own for that run), and attention that reads the cache the first attention run wrote."""

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        H, V = self.d["hidden_size"], self.d["vocab_size"]
        norm = lambda p: PartSpec("rmsnorm", p, {"size": H, "eps": 1e-5})
        ffn = lambda p: PartSpec("swiglu", p, {"hidden_size": H, "intermediate_size": 2 * H})
        rope = {"kind": "rope", "head_dim": 32, "rotary_dim": 32, "theta": 1e4, "layout": "split_half"}
        att = lambda p, kvp: PartSpec("attention", p, {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 32,
                                                       "window": None, "position": rope, "kv_proj": kvp})
        layers = [LayerSpec("prenorm", PartSpec(self.d.get("decay_kind", "test_decay"), "l0.mix", {"hidden_size": H, "decay": 0.9}), ffn("l0.mlp"), norm("l0.n1"), norm("l0.n2")),
                  LayerSpec("prenorm", att("l1.att", True), ffn("l1.mlp"), norm("l1.n1"), norm("l1.n2")),
                  LayerSpec("prenorm", att("l2.att", False), ffn("l2.mlp"), norm("l2.n1"), norm("l2.n2"))]
        return ModelSpec(H, V, 256, layers, [RunSpec(0), RunSpec(1), RunSpec(0), RunSpec(2, cache_of=1)],
                         norm("final"), "embed", None)


def toy_reference(ws, tokens, H):
    x = ws["embed"].double()[torch.tensor(tokens)]
    T = len(tokens)
    rope = {"rotary_dim": 32, "theta": 1e4, "layout": "split_half"}
    inv = plain_inv_freq(32, 1e4, None)
    pos = torch.arange(T)
    shared = {}

    def mlp(x, p):
        xn = plain_rmsnorm(x, ws[f"{p}.n2.weight"].double(), 1e-5)
        return x + plain_swiglu(xn, ws[f"{p}.mlp.gate_proj.weight"].double(), ws[f"{p}.mlp.up_proj.weight"].double(), ws[f"{p}.mlp.down_proj.weight"].double())

    def decay(x):
        xn = plain_rmsnorm(x, ws["l0.n1.weight"].double(), 1e-5)
        s, ys = torch.zeros(H, dtype=torch.float64), []
        for t in range(T):
            s = 0.9 * s + xn[t]
            ys.append(s @ ws["l0.mix.w"].double().T)
        return mlp(x + torch.stack(ys), "l0")

    x = decay(x)
    xn = plain_rmsnorm(x, ws["l1.n1.weight"].double(), 1e-5)
    q = plain_rope((xn @ ws["l1.att.q_proj.weight"].double().T).view(T, 2, 32), pos, inv)
    shared["k"] = plain_rope((xn @ ws["l1.att.k_proj.weight"].double().T).view(T, 1, 32), pos, inv)
    shared["v"] = (xn @ ws["l1.att.v_proj.weight"].double().T).view(T, 1, 32)
    x = mlp(x + plain_attention(q, shared["k"], shared["v"]).reshape(T, 64) @ ws["l1.att.o_proj.weight"].double().T, "l1")
    x = decay(x)                                     # the same layer, run again, with a fresh state
    xn = plain_rmsnorm(x, ws["l2.n1.weight"].double(), 1e-5)
    q = plain_rope((xn @ ws["l2.att.q_proj.weight"].double().T).view(T, 2, 32), pos, inv)
    x = mlp(x + plain_attention(q, shared["k"], shared["v"]).reshape(T, 64) @ ws["l2.att.o_proj.weight"].double().T, "l2")
    return plain_rmsnorm(x, ws["final.weight"].double(), 1e-5) @ ws["embed"].double().T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_a_stateful_mixer(dtype):
    register_mixer("test_decay", DecayMixer)
    register_architecture("TestToyForCausalLM", ToyConfig)
    H, V = 40, 90
    cfg = ToyConfig({"architectures": ["TestToyForCausalLM"], "hidden_size": H, "vocab_size": V})
    from llm_rs_amd.engine import Model
    names = Model(cfg.model_spec(), torch.float32, "cpu").tensors()
    assert "l2.att.k_proj.weight" not in names and "l1.att.k_proj.weight" in names
    ws = {n: ((rnd(s.shape, i) * 0.1 + 1) if s.kind == "norm" else rnd(s.shape, i, 0.2)).bfloat16()
          for i, (n, s) in enumerate(sorted(names.items()))}
    eng = Engine(cfg, ws, dtype=dtype, page_size=16, num_pages=32, max_requests=4)
    assert len(eng.cache.groups) == 1 and eng.cache.groups[0].n_layers == 1, "two attention runs share one cache layer"
    assert len(eng.cache.state_tensors) == 2, "each run of the decay layer has a state of its own"
    seqs = {0: torch.randint(0, V, (50,), generator=torch.Generator().manual_seed(1)).tolist(),
            1: torch.randint(0, V, (23,), generator=torch.Generator().manual_seed(2)).tolist()}
    refs = {i: toy_reference(ws, t, H) for i, t in seqs.items()}
    tol = 3e-5 if dtype == "float32" else 2e-2
    # whole, then in portions side by side with the other request, then the slots are used again
    for cuts in ([50], [9, 2, 20, 1, 1, 17]):
        slots = {i: eng.open_request() for i in seqs}
        pos, rows = {0: 0, 1: 0}, {0: [], 1: []}
        for n in cuts:
            entries = []
            for i in seqs:
                m = min(n, len(seqs[i]) - pos[i])
                if m > 0:
                    entries.append((i, StepEntry(slots[i], pos[i], seqs[i][pos[i]:pos[i] + m], list(range(m)))))
            out = eng.step([e for _, e in entries]).double().cpu()
            at = 0
            for i, e in entries:
                rows[i].append(out[at:at + len(e.tokens)]); at += len(e.tokens); pos[i] += len(e.tokens)
        for i in seqs:
            got = torch.cat(rows[i])
            ref = refs[i][:got.shape[0]]
            assert float((got - ref).abs().max()) <= tol * max(float(ref.abs().max()), 1.0), (cuts, i)
            eng.close_request(slots[i])
    assert eng.generate([seqs[1][:5]], max_new_tokens=4)[0] == eng.generate([seqs[1][:5]], max_new_tokens=4)[0]
    # Through the scheduler, two slots for five requests, one step in flight while the next is planned against
    # stepping in turn: a request that ends on a stop token has run one token more on the device (its state moved
    # once more), and the request that takes its slot must find that state reset.
    prompts = [seqs[0][:7], seqs[1][:3], seqs[0][10:31], seqs[1][5:6], seqs[0][40:44]]
    outs = {}
    for overlap in (False, True):
        small = Engine(cfg, ws, dtype=dtype, page_size=16, num_pages=16, max_requests=2, overlap=overlap)
        free = small.generate(prompts, max_new_tokens=12, temperature=0.8, seed=[1, 2, 3, 4, 5])
        stop = next(t for toks in free for j, t in enumerate(toks) if j >= 2 and t not in toks[:j])
        outs[overlap] = (free, small.generate(prompts, max_new_tokens=12, temperature=0.8, seed=[1, 2, 3, 4, 5],
                                              stop_token_ids=[stop], return_reasons=True))
        assert any(f.reason == "stop" and f.tokens for f in outs[overlap][1]), "the case itself"
    if dtype == "float32":
        assert outs[True][0] == outs[False][0]
        assert [(f.tokens, f.reason) for f in outs[True][1]] == [(f.tokens, f.reason) for f in outs[False][1]]


class RoutedLinear(FeedForward):
    """Each token goes to the expert its router logit is largest for (lowest index on ties):
    y = softmax(x R^T)[e] * (x W_e^T), router logits and softmax in 32-bit."""

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden, self.experts = spec.params["hidden_size"], spec.params["experts"]

    def tensors(self):
        t = {self.name("router"): TensorSpec((self.experts, self.hidden))}
        t.update({self.name(f"expert{e}"): TensorSpec((self.hidden, self.hidden)) for e in range(self.experts)})
        return t

    def load(self, tensors, device):
        self.router = tensors[self.name("router")].to(device=device, dtype=torch.float32)
        self.w = torch.stack([tensors[self.name(f"expert{e}")].to(device=device, dtype=torch.float32) for e in range(self.experts)])

    def forward(self, ctx, x, h):
        xf = x.float()
        p = torch.softmax(xf @ self.router.T, dim=-1)
        e = p.argmax(dim=-1)
        y = torch.einsum("th,toh->to", xf, self.w[e])
        h += y * p.gather(1, e[:, None])


class KeyFade(PositionEncoding):
    """No rotation: the key at position p is scaled by 1 / (1 + p / span), the query is left alone."""

    def __init__(self, params, dtype):
        super().__init__(params, dtype)
        self.span = float(params["span"])

    def apply(self, ctx, q, k):
        if k is not None:
            k.mul_((1.0 / (1.0 + ctx.positions.float() / self.span))[:, None, None].to(k.dtype))


class ToyRoutedConfig:
    """Two layers: attention whose keys fade with their position + a routed feed-forward, then
    rotary attention over a window of 12 keys + SwiGLU."""

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        H, V = self.d["hidden_size"], self.d["vocab_size"]
        norm = lambda p: PartSpec("rmsnorm", p, {"size": H, "eps": 1e-6})
        rope = {"kind": "rope", "head_dim": 16, "rotary_dim": 16, "theta": 1e4, "layout": "split_half"}
        att0 = PartSpec("attention", "l0.att", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 3, "head_dim": 16,
                                                "window": None, "position": {"kind": "test_key_fade", "span": 20.0}})
        att1 = PartSpec("attention", "l1.att", {"hidden_size": H, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                                "window": 12, "position": rope})
        layers = [LayerSpec("prenorm", att0, PartSpec("test_routed", "l0.moe", {"hidden_size": H, "experts": 3}), norm("l0.n1"), norm("l0.n2")),
                  LayerSpec("prenorm", att1, PartSpec("swiglu", "l1.mlp", {"hidden_size": H, "intermediate_size": 3 * H}), norm("l1.n1"), norm("l1.n2"))]
        return ModelSpec(H, V, 256, layers, [RunSpec(0), RunSpec(1)], norm("final"), "embed", "head")


def toy_routed_reference(ws, tokens):
    w = {k: v.double() for k, v in ws.items()}
    x = w["embed"][torch.tensor(tokens)]
    T = len(tokens)
    pos = torch.arange(T)
    xn = plain_rmsnorm(x, w["l0.n1.weight"], 1e-6)
    q = (xn @ w["l0.att.q_proj.weight"].T).view(T, 3, 16)
    k = (xn @ w["l0.att.k_proj.weight"].T).view(T, 3, 16) / (1.0 + pos.double() / 20.0)[:, None, None]
    v = (xn @ w["l0.att.v_proj.weight"].T).view(T, 3, 16)
    x = x + plain_attention(q, k, v).reshape(T, 48) @ w["l0.att.o_proj.weight"].T
    xn = plain_rmsnorm(x, w["l0.n2.weight"], 1e-6)
    p = torch.softmax(xn @ w["l0.moe.router"].T, dim=-1)
    e = p.argmax(dim=-1)
    y = torch.stack([xn[t] @ w[f"l0.moe.expert{int(e[t])}"].T * p[t, e[t]] for t in range(T)])
    x = x + y
    xn = plain_rmsnorm(x, w["l1.n1.weight"], 1e-6)
    inv = plain_inv_freq(16, 1e4, None)
    q = plain_rope((xn @ w["l1.att.q_proj.weight"].T).view(T, 4, 16), pos, inv)
    k = plain_rope((xn @ w["l1.att.k_proj.weight"].T).view(T, 2, 16), pos, inv)
    v = (xn @ w["l1.att.v_proj.weight"].T).view(T, 2, 16)
    x = x + plain_attention(q, k, v, window=12).reshape(T, 64) @ w["l1.att.o_proj.weight"].T
    xn = plain_rmsnorm(x, w["l1.n2.weight"], 1e-6)
    x = x + plain_swiglu(xn, w["l1.mlp.gate_proj.weight"], w["l1.mlp.up_proj.weight"], w["l1.mlp.down_proj.weight"])
    return plain_rmsnorm(x, w["final.weight"], 1e-6) @ w["head"].T, e


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_routing_and_another_position_encoding(dtype):
    register_feed_forward("test_routed", RoutedLinear)
    register_position("test_key_fade", KeyFade)
    register_architecture("TestToyRoutedForCausalLM", ToyRoutedConfig)
    H, V = 56, 77
    cfg = ToyRoutedConfig({"architectures": ["TestToyRoutedForCausalLM"], "hidden_size": H, "vocab_size": V})
    from llm_rs_amd.engine import Model
    names = Model(cfg.model_spec(), torch.float32, "cpu").tensors()
    assert {"l0.moe.router", "l0.moe.expert2", "head"} <= set(names)
    ws = {n: ((rnd(s.shape, i) * 0.1 + 1) if s.kind == "norm" else rnd(s.shape, i, 0.25)).bfloat16()
          for i, (n, s) in enumerate(sorted(names.items()))}
    eng = Engine(cfg, ws, dtype=dtype, page_size=16, num_pages=24, max_requests=4)
    assert len(eng.cache.groups) == 2, "all keys for one layer, a window of them for the other"
    seq = torch.randint(0, V, (60,), generator=torch.Generator().manual_seed(5)).tolist()
    ref, chosen = toy_routed_reference(ws, seq)
    assert len(set(chosen.tolist())) == 3, "the test's tokens should reach every expert"
    tol = 3e-5 if dtype == "float32" else 2.5e-2
    for cuts in ([60], [7, 30, 1, 1, 2, 19]):
        slot, pos, rows = eng.open_request(), 0, []
        for n in cuts:
            rows.append(eng.step([StepEntry(slot, pos, seq[pos:pos + n], list(range(n)))]).double().cpu())
            pos += n
        got = torch.cat(rows)
        if dtype == "float32":
            assert float((got - ref).abs().max()) <= tol * max(float(ref.abs().max()), 1.0), cuts
        else:
            # a token whose two best router logits are close may go to another expert in 16-bit: leave those rows out
            xs = (got - ref).abs().max(dim=1).values <= tol * max(float(ref.abs().max()), 1.0)
            assert int((~xs).sum()) <= 3, (cuts, int((~xs).sum()))
        eng.close_request(slot)


# ---- a stateful mixer whose decode steps may be recorded ----------------------------------------

class RecordableDecayMixer(DecayMixer):
    """The same mixer, with a decode step that launches only device work whose arguments do not
    change between steps of one shape (the rows of the state are found through the slots on the
    device): it says so, and the step function may then record and replay such steps."""
    graph_safe = True

    def forward(self, ctx, x, h, cache):
        if ctx.n_single != ctx.n_entries:
            return super().forward(ctx, x, h, cache)
        slots = ctx.slots.long()
        s = cache.state[slots] * self.decay + x.float()
        cache.state.index_copy_(0, slots, s)
        h += s @ self.w.T


def test_decode_steps_of_a_stateful_mixer_are_recorded_and_replayed():
    register_mixer("test_decay", DecayMixer)
    register_mixer("test_decay_recordable", RecordableDecayMixer)
    register_architecture("TestToyForCausalLM", ToyConfig)
    H, V = 40, 90
    from llm_rs_amd.engine import Model
    cfg = ToyConfig({"architectures": ["TestToyForCausalLM"], "hidden_size": H, "vocab_size": V, "decay_kind": "test_decay_recordable"})
    names = Model(cfg.model_spec(), torch.float32, "cpu").tensors()
    ws = {n: ((rnd(s.shape, i) * 0.1 + 1) if s.kind == "norm" else rnd(s.shape, i, 0.2)).bfloat16()
          for i, (n, s) in enumerate(sorted(names.items()))}
    eng = Engine(cfg, ws, dtype="float32", page_size=16, num_pages=32, max_requests=4)
    assert eng.runner.use_graphs, "fixed-size state does not keep a model whose parts are all graph_safe from being recorded"
    plain = Engine(ToyConfig({**cfg.d, "decay_kind": "test_decay"}), ws, dtype="float32", page_size=16, num_pages=32, max_requests=4)
    assert not plain.runner.use_graphs, "a part that does not say graph_safe keeps the whole model eager"
    seqs = {0: torch.randint(0, V, (40,), generator=torch.Generator().manual_seed(1)).tolist(),
            1: torch.randint(0, V, (40,), generator=torch.Generator().manual_seed(2)).tolist()}
    refs = {i: toy_reference(ws, t, H) for i, t in seqs.items()}
    for round_ in range(2):                              # the second round reuses the slots: their state starts from zero again
        slots = {i: eng.open_request() for i in seqs}
        rows = {0: [], 1: []}
        out = eng.step([StepEntry(slots[i], 0, seqs[i][:6], [5]) for i in seqs]).double().cpu()   # a prompt portion first
        for i in seqs:
            rows[i].append(out[i])
        for p in range(6, 40):
            out = eng.step([StepEntry(slots[i], p, [seqs[i][p]], [0]) for i in seqs]).double().cpu()
            for i in seqs:
                rows[i].append(out[i])
        for i in seqs:
            got, ref = torch.stack(rows[i]), refs[i][5:]
            assert float((got - ref).abs().max()) <= 3e-5 * max(float(ref.abs().max()), 1.0), (round_, i)
            eng.close_request(slots[i])
    assert eng.runner.graph_replays >= 60, eng.runner.graph_replays


class KeyedDecayMixer(RecordableDecayMixer):
    """The same again, but what a decode step launches follows a host value that moves from step to step though
    the step's sizes stay (here: whether the requests' lengths add up to an even number of fours): the part names
    what that depends on and what it comes to for a step, and the step function keeps a recording for each value."""
    recording_signature = "test_keyed_decay"

    def recording_key(self, ctx):
        return (sum(ctx.single_lens) // 4) % 2

    def forward(self, ctx, x, h, cache):
        super().forward(ctx, x, h, cache)
        if ctx.n_single == ctx.n_entries and self.recording_key(ctx):
            h += 0.25


def test_a_part_whose_launches_follow_a_host_value_gets_a_recording_for_each_value():
    register_mixer("test_decay_keyed", KeyedDecayMixer)
    register_architecture("TestToyForCausalLM", ToyConfig)
    H, V = 40, 90
    from llm_rs_amd.engine import Model
    cfg = ToyConfig({"architectures": ["TestToyForCausalLM"], "hidden_size": H, "vocab_size": V, "decay_kind": "test_decay_keyed"})
    names = Model(cfg.model_spec(), torch.float32, "cpu").tensors()
    ws = {n: ((rnd(s.shape, i) * 0.1 + 1) if s.kind == "norm" else rnd(s.shape, i, 0.2)).bfloat16()
          for i, (n, s) in enumerate(sorted(names.items()))}
    recorded = Engine(cfg, ws, dtype="float32", page_size=16, num_pages=32, max_requests=4)
    eager = Engine(cfg, ws, dtype="float32", page_size=16, num_pages=32, max_requests=4)
    eager.runner.use_graphs = False
    assert recorded.runner.use_graphs
    seqs = [torch.randint(0, V, (40,), generator=torch.Generator().manual_seed(5 + i)).tolist() for i in range(2)]
    slots = {eng: [eng.open_request() for _ in seqs] for eng in (recorded, eager)}
    for eng in (recorded, eager):
        eng.step([StepEntry(slots[eng][i], 0, seqs[i][:6], []) for i in range(2)])
    with_it = 0
    for p in range(6, 40):
        a, b = (eng.step([StepEntry(slots[eng][i], p, [seqs[i][p]], [0]) for i in range(2)]).clone() for eng in (recorded, eager))
        torch.cuda.synchronize()
        assert torch.equal(a, b), f"position {p}"
        with_it += ((2 * (p + 1)) // 4) % 2
    assert 10 <= with_it <= 24, "the case itself: both values come"
    assert len(recorded.runner._graphs) == 2 and recorded.runner.graph_replays >= 28


# ---- other arrangements of a layer, a scaled embedding and bent logits ---------------------------

class ParallelBlock(Block):
    """One norm feeds both halves: x = norm(h); h += mixer(x); h += feed_forward(x)."""
    needs = ("mixer", "feed_forward", "mixer_norm")

    def forward(self, ctx, h, cache):
        x = ctx.workspace("block.x", tuple(h.shape), self.mixer.dtype)
        self.mixer_norm.forward(ctx, h, x)
        self.mixer.forward(ctx, x, h, cache)
        self.feed_forward.forward(ctx, x, h)


class SandwichBlock(Block):
    """A norm before and a norm after each half: h += post(mixer(pre(h))); the same for the feed-forward.
    The two norms after come as the layer spec's extra parts."""
    needs = ("mixer", "feed_forward", "mixer_norm", "feed_forward_norm", "post_mixer_norm", "post_feed_forward_norm")

    def _half(self, ctx, h, pre, part, post, *cache):
        x = ctx.workspace("block.x", tuple(h.shape), self.mixer.dtype)
        pre.forward(ctx, h, x)
        t = ctx.workspace("sandwich.t", tuple(h.shape), torch.float32)
        t.zero_()
        part.forward(ctx, x, t, *cache)                  # parts add into the stream they are given
        post.forward(ctx, t, x)
        h += x.float()

    def forward(self, ctx, h, cache):
        self._half(ctx, h, self.mixer_norm, self.mixer, self.named["post_mixer_norm"], cache)
        self._half(ctx, h, self.feed_forward_norm, self.feed_forward, self.named["post_feed_forward_norm"])


class ToyShapesConfig:
    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        H, V = self.d["hidden_size"], self.d["vocab_size"]
        norm = lambda p: PartSpec("rmsnorm", p, {"size": H, "eps": 1e-5})
        ffn = lambda p: PartSpec("swiglu", p, {"hidden_size": H, "intermediate_size": 2 * H})
        rope = {"kind": "rope", "head_dim": 16, "rotary_dim": 16, "theta": 1e4, "layout": "split_half"}
        att = lambda p: PartSpec("attention", p, {"hidden_size": H, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                                  "window": None, "position": rope})
        layers = [LayerSpec("test_parallel", mixer=att("l0.att"), feed_forward=ffn("l0.mlp"), mixer_norm=norm("l0.n")),
                  LayerSpec("test_sandwich", att("l1.att"), ffn("l1.mlp"), norm("l1.n1"), norm("l1.n2"),
                            extra=(ExtraPart("post_mixer_norm", "norm", norm("l1.n1post")),
                                   ExtraPart("post_feed_forward_norm", "norm", norm("l1.n2post"))))]
        return ModelSpec(H, V, 256, layers, [RunSpec(0), RunSpec(1)], norm("final"), "embed", None,
                         embedding_scale=math.sqrt(H), logit_scale=0.5, logit_softcap=4.0)


def toy_shapes_reference(ws, tokens, H):
    w = {k: v.double() for k, v in ws.items()}
    T = len(tokens)
    pos = torch.arange(T)
    inv = plain_inv_freq(16, 1e4, None)
    x = w["embed"][torch.tensor(tokens)] * float(torch.tensor(math.sqrt(H), dtype=torch.float32))

    def att(xn, p):
        q = plain_rope((xn @ w[f"{p}.q_proj.weight"].T).view(T, 4, 16), pos, inv)
        k = plain_rope((xn @ w[f"{p}.k_proj.weight"].T).view(T, 2, 16), pos, inv)
        v = (xn @ w[f"{p}.v_proj.weight"].T).view(T, 2, 16)
        return plain_attention(q, k, v).reshape(T, 64) @ w[f"{p}.o_proj.weight"].T

    mlp = lambda xn, p: plain_swiglu(xn, w[f"{p}.gate_proj.weight"], w[f"{p}.up_proj.weight"], w[f"{p}.down_proj.weight"])
    n = lambda x, name: plain_rmsnorm(x, w[f"{name}.weight"], 1e-5)
    xn = n(x, "l0.n")
    x = x + att(xn, "l0.att") + mlp(xn, "l0.mlp")
    x = x + n(att(n(x, "l1.n1"), "l1.att"), "l1.n1post")
    x = x + n(mlp(n(x, "l1.n2"), "l1.mlp"), "l1.n2post")
    logits = n(x, "final") @ w["embed"].T * 0.5
    return 4.0 * torch.tanh(logits / 4.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_other_block_arrangements_scaled_embedding_and_bent_logits(dtype):
    register_block("test_parallel", ParallelBlock)
    register_block("test_sandwich", SandwichBlock)
    register_architecture("TestToyShapesForCausalLM", ToyShapesConfig)
    H, V = 64, 101
    cfg = ToyShapesConfig({"architectures": ["TestToyShapesForCausalLM"], "hidden_size": H, "vocab_size": V})
    from llm_rs_amd.engine import Model
    probe = Model(cfg.model_spec(), torch.float32, "cpu")
    names = probe.tensors()
    assert {"l0.n.weight", "l1.n1post.weight", "l1.n2post.weight"} <= set(names) and "l0.n2.weight" not in names
    with pytest.raises(ValueError, match="needs the parts"):
        build_block(LayerSpec("test_sandwich", cfg.model_spec().layers[1].mixer), torch.float32)
    ws = {n: ((rnd(s.shape, i) * 0.1 + 1) if s.kind == "norm" else rnd(s.shape, i, 0.2)).bfloat16()
          for i, (n, s) in enumerate(sorted(names.items()))}
    eng = Engine(cfg, ws, dtype=dtype, page_size=16, num_pages=24, max_requests=4)
    assert eng.model.weight_bytes_per_step() == sum(t.numel() * (4 if dtype == "float32" or n.endswith(".weight") and t.dim() == 1 else 2)
                                                    for n, t in ws.items())
    back = eng.weights()
    assert all(torch.equal(back[n].float(), t.float()) for n, t in ws.items()), "every part gives its tensors back"
    seq = torch.randint(0, V, (50,), generator=torch.Generator().manual_seed(8)).tolist()
    ref = toy_shapes_reference(ws, seq, H)
    assert float(ref.abs().max()) < 4.0 and float(ref.abs().max()) > 1.0, "the cap must bite for the test to see it"
    tol = 3e-5 if dtype == "float32" else 2e-2
    for cuts in ([50], [9, 2, 20, 1, 1, 17]):
        slot, pos, rows = eng.open_request(), 0, []
        for n in cuts:
            rows.append(eng.step([StepEntry(slot, pos, seq[pos:pos + n], list(range(n)))]).double().cpu())
            pos += n
        got = torch.cat(rows)
        assert float((got - ref).abs().max()) <= tol * max(float(ref.abs().max()), 1.0), cuts
        eng.close_request(slot)


# ---- a mixer with a cache kind of its own, a family of parts of its own, and no final norm -------------------------

from dataclasses import dataclass  # noqa: E402

from llm_rs_amd.cache import CacheKind, CacheView, register_cache_kind  # noqa: E402
from llm_rs_amd.parts import Part, register_part_family  # noqa: E402


@dataclass(frozen=True)
class PagedLatent:
    """One vector of `width` numbers per token, in pages."""
    width: int
    window: int = 0


class PagedLatentKind(CacheKind):
    """[layer][page][slot][width] in 32-bit, whatever the engine computes in."""
    paged = True

    def window(self, need):
        return need.window

    def bytes_per_token(self, need, dtype):
        return 4 * need.width

    def allocate_pages(self, need, n_layers, num_pages, page_size, dtype, device):
        return torch.zeros((n_layers, num_pages, page_size, need.width), dtype=torch.float32, device=device)

    def page_view(self, storage, need, layer, group, page_size, num_pages, writes):
        return CacheView("latent", group, page_size=page_size, num_pages=num_pages, writes=writes, data=storage[layer])


class LatentMixer(Mixer):
    """c_t = x_t Wc^T is what a token leaves in the cache; y_t = (sum_j<=t softmax_j((x_t Wq^T) . c_j / sqrt(L)) c_j) Wo^T:
    attention whose keys and values are the same latent vector."""

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden, self.width = spec.params["hidden_size"], spec.params["latent"]

    def tensors(self):
        return {self.name("c"): TensorSpec((self.width, self.hidden)), self.name("q"): TensorSpec((self.width, self.hidden)),
                self.name("o"): TensorSpec((self.hidden, self.width))}

    def load(self, tensors, device):
        self.wc, self.wq, self.wo = (tensors[self.name(n)].to(device=device, dtype=torch.float32) for n in "cqo")

    def export(self):
        return {self.name(n): w.cpu() for n, w in zip("cqo", (self.wc, self.wq, self.wo))}

    def cache_need(self):
        return PagedLatent(self.width)

    def forward(self, ctx, x, h, cache):
        assert cache.kind == "latent" and cache.data.shape[1:] == (cache.page_size, self.width)
        g, L = cache.group, self.width
        xf = x.float()
        cache.data.view(-1, L)[ctx.slot_maps[g].long()] = xf @ self.wc.T       # this step's latents into their pages
        at = 0
        for e, (slot, start, count) in enumerate(ctx.entries):
            n = start + count
            pages = ctx.block_tables[g][e, :-(-n // cache.page_size)].long()
            lat = cache.data[pages].reshape(-1, L)[:n]                          # the request's latents, in order
            s = (xf[at:at + count] @ self.wq.T) @ lat.T / math.sqrt(L)
            seen = torch.arange(n, device=s.device)[None, :] <= (start + torch.arange(count, device=s.device))[:, None]
            p = torch.softmax(s.masked_fill(~seen, -math.inf), dim=-1)
            h[at:at + count] += (p @ lat) @ self.wo.T
            at += count


class VectorGate(Part):
    """A part that is neither mixer, feed-forward nor norm: one number per feature."""

    def tensors(self):
        return {self.name("g"): TensorSpec((self.spec.params["size"],))}

    def load(self, tensors, device):
        self.g = tensors[self.name("g")].to(device=device, dtype=torch.float32)

    def export(self):
        return {self.name("g"): self.g.cpu()}


class GatedBlock(Block):
    """h += mixer(norm(h)); h += gate * feed_forward(norm(h)), the gate a part of a family of its own."""
    needs = ("mixer", "feed_forward", "mixer_norm", "feed_forward_norm", "gate")

    def forward(self, ctx, h, cache):
        self.mixer.forward(ctx, self.normed_input(ctx, h, self.mixer_norm, self.mixer, None), h, cache)
        x = self.normed_input(ctx, h, self.feed_forward_norm, self.feed_forward, None)
        y = torch.zeros_like(h)
        self.feed_forward.forward(ctx, x, y)
        h += y * self.named["gate"].g
        ctx.note_left(h, None)


class ToyLatentConfig:
    """Two layers: the latent mixer in a gated block, then grouped-query attention in the usual block; no norm
    between the last block and the output matrix."""

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        H, V = self.d["hidden_size"], self.d["vocab_size"]
        norm = lambda p: PartSpec("rmsnorm", p, {"size": H, "eps": 1e-5})
        ffn = lambda p: PartSpec("swiglu", p, {"hidden_size": H, "intermediate_size": 2 * H})
        rope = {"kind": "rope", "head_dim": 32, "rotary_dim": 32, "theta": 1e4, "layout": "split_half"}
        att = PartSpec("attention", "l1.att", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 32, "window": None, "position": rope})
        layers = [LayerSpec("test_gated", PartSpec("test_latent", "l0.mix", {"hidden_size": H, "latent": 24}), ffn("l0.mlp"), norm("l0.n1"), norm("l0.n2"),
                            extra=(ExtraPart("gate", "test_gate", PartSpec("vector", "l0.gate", {"size": H})),)),
                  LayerSpec("prenorm", att, ffn("l1.mlp"), norm("l1.n1"), norm("l1.n2"))]
        return ModelSpec(H, V, 512, layers, [RunSpec(0), RunSpec(1)], None, "embed", "head")


def toy_latent_reference(ws, tokens, r=lambda t: t):
    """`r`: applied to what one kernel hands the next (the identity for the exact result; rounding to bfloat16 to see
    what rounding alone does to these logits)."""
    w = {k: v.double() for k, v in ws.items()}
    T = len(tokens)
    x = w["embed"][torch.tensor(tokens)]
    mlp = lambda xn, p: plain_swiglu(xn, w[f"{p}.gate_proj.weight"], w[f"{p}.up_proj.weight"], w[f"{p}.down_proj.weight"], r)
    xn = r(plain_rmsnorm(x, w["l0.n1.weight"], 1e-5))
    c, q = xn @ w["l0.mix.c"].T, xn @ w["l0.mix.q"].T             # (the toy mixer computes in 32-bit from the normed rows)
    s = (q @ c.T / math.sqrt(24)).masked_fill(torch.ones(T, T).triu(1).bool(), -math.inf)
    x = x + (torch.softmax(s, dim=-1) @ c) @ w["l0.mix.o"].T
    x = x + w["l0.gate.g"] * mlp(r(plain_rmsnorm(x, w["l0.n2.weight"], 1e-5)), "l0.mlp")
    xn = r(plain_rmsnorm(x, w["l1.n1.weight"], 1e-5))
    pos, inv = torch.arange(T), plain_inv_freq(32, 1e4, None)
    qq = r(plain_rope((xn @ w["l1.att.q_proj.weight"].T).view(T, 2, 32), pos, inv))
    kk = r(plain_rope((xn @ w["l1.att.k_proj.weight"].T).view(T, 1, 32), pos, inv))
    vv = r((xn @ w["l1.att.v_proj.weight"].T).view(T, 1, 32))
    x = x + r(plain_attention(qq, kk, vv, rounded=r).reshape(T, 64)) @ w["l1.att.o_proj.weight"].T
    x = x + mlp(r(plain_rmsnorm(x, w["l1.n2.weight"], 1e-5)), "l1.mlp")
    return r(x) @ w["head"].T                                      # no final norm


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_a_cache_kind_of_its_own(dtype):
    """A need of a class the package has never seen (one latent vector per token, paged), a family of parts it has
    never seen, and a stack without a final norm: registered here, sized, paged, given back and replayed in the four
    cuts (whole, the tail token by token, portions, mixed with so few pages that they are used again) by the cache
    manager, step function and trace replay as they are."""
    from llm_rs_amd.engine import Model
    from llm_rs_amd.engine.trace import TraceReplayer
    from replay_cases import live_token_need, mixed, portions, tail_decoded, whole
    from replay_checks import check_rows, run_trace
    register_cache_kind(PagedLatent, PagedLatentKind())
    register_mixer("test_latent", LatentMixer)
    register_part_family("test_gate")("vector", VectorGate)
    register_block("test_gated", GatedBlock)
    register_architecture("TestToyLatentForCausalLM", ToyLatentConfig)
    H, V = 48, 83
    cfg = ToyLatentConfig({"architectures": ["TestToyLatentForCausalLM"], "hidden_size": H, "vocab_size": V})
    names = Model(cfg.model_spec(), torch.float32, "cpu").tensors()
    assert {"l0.gate.g", "l0.mix.c", "head"} <= set(names) and "final.weight" not in names
    ws = {n: ((rnd(s.shape, i) * 0.1 + 1) if s.kind == "norm" else rnd(s.shape, i, 0.2)).bfloat16()
          for i, (n, s) in enumerate(sorted(names.items()))}
    with pytest.raises(TypeError, match="registered class"):
        CacheManager([(("keys", 3), None)], torch.float32, DEV, 16, 4, max_requests=2)
    # what the pool is sized by is the kinds' to say: 24 floats a token for the latents, 2 x 32 values for the keys and values
    per_token = 4 * 24 + 2 * 32 * (4 if dtype == "float32" else 2)
    needs = Model(cfg.model_spec(), torch.float32, "cpu").cache_needs()
    assert needs[0][0] == PagedLatent(24)
    assert CacheManager.pages_that_fit(needs, torch.float32 if dtype == "float32" else torch.bfloat16, 16, 10_000_000, 0.5, 64, 512) \
        == [min(5_000_000 // per_token, 64 * 512) // 16] * 2
    requests = {f"r{i}": torch.randint(0, V, (n,), generator=torch.Generator().manual_seed(30 + i)).tolist()
                for i, n in enumerate((70, 41, 100, 33, 57))}
    reference = {rid: toy_latent_reference(ws, toks) for rid, toks in requests.items()}
    # bfloat16: as for the real models, the bound is made from what rounding between kernels alone does to these logits
    to_bf16 = lambda t: t.to(torch.bfloat16).to(t.dtype)
    by_rounding = max(float((toy_latent_reference(ws, toks, to_bf16) - reference[rid]).abs().max()) / float(reference[rid].abs().max())
                      for rid, toks in requests.items())
    allowed = 3e-5 if dtype == "float32" else 1.5 * by_rounding
    for name, steps in (("whole", whole(requests)), ("tail", tail_decoded(requests, 32)), ("portions", portions(requests)),
                        ("mixed", mixed(requests, live=3))):
        need = live_token_need(steps)
        eng = Engine(cfg, ws, dtype=dtype, page_size=16, num_pages=need // 16, max_requests=8)
        assert len(eng.cache.groups) == 2 and eng.cache.bytes_per_token() == per_token
        assert eng.cache.views[0].kind == "latent" and eng.cache.views[1].kind == "paged" and eng.model.final_norm is None
        rows, _ = run_trace(lambda n: TraceReplayer.for_engine(eng), steps)
        check_rows(rows, reference, dtype, requests, allowed)
        core = eng.cache.core
        assert all(core.pages_free(g) == core.pages_total(g) for g in range(2)) and core.slots_in_use() == 0, name
    back = eng.weights()
    assert all(torch.equal(back[n].float(), t.float()) for n, t in ws.items())
    out = eng.generate([requests["r1"][:9]], max_new_tokens=5)[0]
    assert len(out) == 5
    if dtype == "float32":
        full = toy_latent_reference(ws, requests["r1"][:9] + out)
        assert out == [int(full[8 + i].argmax()) for i in range(5)]
