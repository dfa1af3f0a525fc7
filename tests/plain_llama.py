"""A plain, slow Llama decoder for the tests to compare the engine with.

Whole sequences, no cache, no batching, one function for each part, written from
the reference's formulas (each function cites them) in ordinary tensor
operations.  It shares no code with the package: it reads config.json and
model.safetensors itself.  Computation is in the dtype of `compute` (float64 by
default) from the weights as stored.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional, Sequence

import torch

_ST_DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64}


def read_model_folder(folder: str):
    """(config dict, {name: tensor}) read directly from the files."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    for name, e in header.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        t = torch.frombuffer(bytearray(data[lo:hi]), dtype=_ST_DTYPES[e["dtype"]]).reshape(e["shape"])
        tensors[name] = t.clone()
    return cfg, tensors


# ---- parts -------------------------------------------------------------------

def plain_embedding(table: torch.Tensor, tokens: Sequence[int]) -> torch.Tensor:
    """x[t, :] = table[tok[t], :], no scaling (src/arch/llama.rs:150, shaders/ops.metal:878-902)."""
    return table[torch.tensor(list(tokens), dtype=torch.long, device=table.device)]


def plain_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """ss = sum x^2; inv = rsqrt(ss / D + eps); y = x * inv * w; the weight
    multiplies directly (shaders/ops.metal:980-1002)."""
    ss = (x * x).sum(dim=-1, keepdim=True)
    inv = 1.0 / torch.sqrt(ss / x.shape[-1] + eps)
    return x * inv * w


def plain_inv_freq(rotary_dim: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """freq_i = 1 / theta^(2i/d) (shaders/ops.metal:1030).  The reference scales
    nothing; "llama3" scaling follows the engine's own statement of it: by
    wavelength 2 pi / freq against L = original_max_position_embeddings: shorter
    than L/high kept, longer than L/low divided by factor, between blended linearly
    in L/wavelength.  Rounded to float32, as the engine's table is."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    freq = 1.0 / (theta ** (2.0 * i / rotary_dim))
    if scaling is not None and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor, low, high = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
        L = scaling["original_max_position_embeddings"]
        wavelength = 2.0 * math.pi / freq
        smooth = (L / wavelength - low) / (high - low)
        blended = (1.0 - smooth) * freq / factor + smooth * freq
        freq = torch.where(wavelength < L / high, freq, torch.where(wavelength > L / low, freq / factor, blended))
    return freq.to(torch.float32)


def plain_rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, layout: str = "split_half") -> torch.Tensor:
    """x: [T, heads, head_dim].  angle = float(pos) * freq_i in 32-bit;
    (a, b) <- (a cos - b sin, a sin + b cos) (shaders/ops.metal:1031-1041); the pair
    is (i, i + d/2) for "split_half", (2i, 2i+1) for "interleaved"
    (src/tensor/mod.rs:133-139).  Features past the rotary width are unchanged."""
    rot = 2 * inv_freq.shape[0]
    angle = (positions.to(torch.float32)[:, None] * inv_freq[None, :]).to(device=x.device, dtype=x.dtype)   # [T, rot/2]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    out = x.clone()
    if layout == "split_half":
        a, b = x[..., :rot // 2], x[..., rot // 2:rot]
        out[..., :rot // 2] = a * cos - b * sin
        out[..., rot // 2:rot] = a * sin + b * cos
    elif layout == "interleaved":
        a, b = x[..., 0:rot:2], x[..., 1:rot:2]
        out[..., 0:rot:2] = a * cos - b * sin
        out[..., 1:rot:2] = a * sin + b * cos
    else:
        raise ValueError(layout)
    return out


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None,
                    window: int = 0, positions: Optional[torch.Tensor] = None, rounded=lambda t: t) -> torch.Tensor:
    """q: [T, heads, d]; k, v: [T, kv_heads, d]; one sequence, causal.
    Head h uses kv head h / (heads / kv_heads); s_j = (q . k_j) * rsqrt(d), the scale
    after the dot; keys j <= the query's place (and > place - window if a window is
    given); softmax over j; o = sum_j p_j v_j (shaders/ops.metal:658-757).
    (`rounded`: see `plain_forward_streamed`; applied to the probabilities.)"""
    T, H, d = q.shape
    KV = k.shape[1]
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.zeros_like(q)
    place = (torch.arange(T) if positions is None else positions).to(q.device)
    for h in range(H):
        g = h // (H // KV)
        scores = (q[:, h, :] @ k[:, g, :].T) * scale                      # [T, T]
        visible = place[None, :] <= place[:, None]
        if window > 0:
            visible &= place[None, :] > place[:, None] - window
        scores = scores.masked_fill(~visible, float("-inf"))
        out[:, h, :] = rounded(torch.softmax(scores, dim=-1)) @ v[:, g, :]
    return out


def plain_silu(x: torch.Tensor) -> torch.Tensor:
    """v / (1 + exp(-v)) (shaders/ops.metal:769)."""
    return x / (1.0 + torch.exp(-x))


def plain_swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, rounded=lambda t: t) -> torch.Tensor:
    """(silu(x Wg^T) * (x Wu^T)) Wd^T (src/arch/llama.rs:165-169).  (`rounded`: see `plain_forward_streamed`.)"""
    return rounded(plain_silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


# ---- the model -----------------------------------------------------------------

def plain_layer(cfg: dict, W: Dict[str, torch.Tensor], prefix: str, x: torch.Tensor, pos: torch.Tensor,
                inv_freq: torch.Tensor, layout: str = "split_half", rounded=lambda t: t) -> torch.Tensor:
    """One layer on one whole sequence x [T, hidden]: x += attention(norm(x)); x += swiglu(norm(x))
    (src/arch/llama.rs:151-170).  `W` holds the layer's tensors under `prefix` + their names.
    (`rounded`: see `plain_forward_streamed`.)"""
    H, D = cfg["num_attention_heads"], cfg["hidden_size"]
    KV = cfg.get("num_key_value_heads") or H
    d = cfg.get("head_dim") or D // H
    eps = cfg.get("rms_norm_eps", 1e-5)
    T = x.shape[0]
    p = prefix
    r = rounded
    xn = r(plain_rmsnorm(x, W[p + "input_layernorm.weight"], eps))
    q = (xn @ W[p + "self_attn.q_proj.weight"].T).view(T, H, d)
    k = (xn @ W[p + "self_attn.k_proj.weight"].T).view(T, KV, d)
    v = r((xn @ W[p + "self_attn.v_proj.weight"].T).view(T, KV, d))
    q, k = r(plain_rope(q, pos, inv_freq, layout)), r(plain_rope(k, pos, inv_freq, layout))
    o = r(plain_attention(q, k, v, rounded=r).reshape(T, H * d))
    x = x + o @ W[p + "self_attn.o_proj.weight"].T
    xn = r(plain_rmsnorm(x, W[p + "post_attention_layernorm.weight"], eps))
    return x + plain_swiglu(xn, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"], r)


def plain_forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int],
                  compute: torch.dtype = torch.float64, layout: str = "split_half",
                  position_offset: int = 0) -> torch.Tensor:
    """Logits [T, vocab] for one whole sequence from position 0 (or `position_offset`).  Layer loop of
    src/arch/llama.rs:150-171, final norm and output matrix of :135-139; tied
    embeddings reuse the token table (:81)."""
    return plain_forward_streamed(cfg, lambda name: weights[name], [tokens], compute, layout, position_offset)[0]


def plain_forward_streamed(cfg: dict, tensor_of, sequences: Sequence[Sequence[int]], compute: torch.dtype = torch.float64,
                           layout: str = "split_half", position_offset: int = 0, rows: Optional[Sequence[Sequence[int]]] = None,
                           rounding: Optional[torch.dtype] = None, device="cpu", also_in: Optional[torch.dtype] = None):
    """The same for several whole sequences, one after the other through each layer, with the
    tensors asked for by name through `tensor_of(name)` when their layer is reached and dropped
    after it: a model too large to hold in `compute` precision needs one layer's worth of room.
    `rows[i]`: the places of sequence i whose logits are wanted (default: all).  `device`: where the
    tensor operations run (the same plain operations; a long sequence through a deep model takes
    minutes on the host).
    `rounding`: a second pass beside the first in which every activation that a kernel of an engine
    computing in that type hands to the next kernel through memory is rounded to it (the normed rows,
    q, k and v, the probabilities, the attention's output, silu(gate) * up, the output matrix's input;
    never the residual stream, never a sum).  It says how far rounding alone takes this model on these
    sequences from the exact result; the return value is then (logits, logits of the rounded pass)."""
    H, D = cfg["num_attention_heads"], cfg["hidden_size"]
    d = cfg.get("head_dim") or D // H
    inv_freq = plain_inv_freq(d, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    get = lambda name: tensor_of(name).to(device)
    rounded = (lambda t: t.to(rounding).to(t.dtype)) if rounding is not None else None
    table = get("model.embed_tokens.weight")
    xs = [plain_embedding(table, tokens).to(compute) for tokens in sequences]
    ys = [x.clone() for x in xs] if rounded else None
    zs = [x.to(also_in) for x in xs] if also_in is not None else None
    positions = [torch.arange(len(tokens)) + position_offset for tokens in sequences]
    leaves = ("input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight",
              "self_attn.o_proj.weight", "post_attention_layernorm.weight", "mlp.gate_proj.weight", "mlp.up_proj.weight",
              "mlp.down_proj.weight")
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        W = {p + leaf: get(p + leaf).to(compute) for leaf in leaves}
        xs = [plain_layer(cfg, W, p, x, pos, inv_freq, layout) for x, pos in zip(xs, positions)]
        if rounded:
            ys = [plain_layer(cfg, W, p, y, pos, inv_freq, layout, rounded) for y, pos in zip(ys, positions)]
        if zs is not None:
            W = {n: t.to(also_in) for n, t in W.items()}
            zs = [plain_layer(cfg, W, p, z, pos, inv_freq, layout) for z, pos in zip(zs, positions)]
        del W
    norm = get("model.norm.weight").to(compute)
    head = (table if cfg.get("tie_word_embeddings", False) else get("lm_head.weight")).to(compute)
    eps = cfg.get("rms_norm_eps", 1e-5)
    pick = lambda x, i: x if rows is None else x[torch.tensor(list(rows[i]), dtype=torch.long, device=x.device)]
    exact = [plain_rmsnorm(pick(x, i), norm, eps) @ head.T for i, x in enumerate(xs)]
    if not rounded and zs is None:
        return exact
    out = [exact]
    if rounded:
        out.append([rounded(plain_rmsnorm(pick(y, i), norm, eps)) @ head.T for i, y in enumerate(ys)])
    if zs is not None:
        norm, head = norm.to(also_in), head.to(also_in)
        out.append([plain_rmsnorm(pick(z, i), norm, eps) @ head.T for i, z in enumerate(zs)])
    return tuple(out)


# ---- sampling ------------------------------------------------------------------

class PlainXorshift:
    """xorshift64 with shifts 13, 7, 17; seed 0 stands for 0xDEADBEEFCAFE; a float is
    the top 24 bits over 2^24 (src/sampler/mod.rs:7-24)."""

    def __init__(self, seed: int):
        self.state = 0xDEADBEEFCAFE if seed == 0 else seed

    def next_u64(self) -> int:
        x = self.state
        x ^= (x << 13) & 0xFFFFFFFFFFFFFFFF
        x ^= x >> 7
        x ^= (x << 17) & 0xFFFFFFFFFFFFFFFF
        self.state = x
        return x

    def next_f32(self) -> float:
        return (self.next_u64() >> 40) / float(1 << 24)


def plain_argmax(logits: torch.Tensor) -> int:
    """Greedy; of equal logits the lowest index (the engine's rule; the reference
    leaves ties open, shaders/ops.metal:803-835 vs src/sampler/mod.rs:65-68)."""
    best = logits.max()
    return int((logits == best).nonzero()[0])


def plain_probabilities(logits: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """The distribution the reference samples from (src/sampler/mod.rs:84-141), in
    float64: logits / T; all but the top_k largest dropped; softmax; the smallest
    prefix of the descending order whose mass reaches top_p kept and renormalised.
    Ties at a cut are broken towards the lower index (the reference's unstable
    sorts leave them open)."""
    z = logits.to(torch.float64) * (1.0 / temperature)
    V = z.shape[0]
    order = sorted(range(V), key=lambda i: (-float(z[i]), i))
    keep = torch.ones(V, dtype=torch.bool)
    if 0 < top_k < V:
        keep[:] = False
        keep[order[:top_k]] = True
    z = z.masked_fill(~keep, float("-inf"))
    p = torch.softmax(z, dim=0)
    if top_p < 1.0:
        total, cut = 0.0, V
        for n, i in enumerate(order):
            total += float(p[i])
            if total >= top_p:
                cut = n + 1
                break
        drop = order[cut:]
        p[drop] = 0.0
        p = p / p.sum()
    return p


def plain_sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, rng: PlainXorshift) -> int:
    """One draw: the first index whose cumulative probability exceeds the uniform,
    walking in index order (src/sampler/mod.rs:143-154)."""
    if temperature == 0.0:
        return plain_argmax(logits)
    p = plain_probabilities(logits, temperature, top_k, top_p)
    r = rng.next_f32()
    cum = torch.cumsum(p, dim=0)
    hit = (cum > r).nonzero()
    return int(hit[0]) if len(hit) else int(p.nonzero()[-1])


def plain_generate(cfg: dict, weights: Dict[str, torch.Tensor], prompt: Sequence[int], max_new: int,
                   temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed: int = 42,
                   stop: Sequence[int] = (), compute: torch.dtype = torch.float64) -> List[int]:
    """The whole sequence is run again for every new token."""
    rng = PlainXorshift(seed)
    tokens, out = list(prompt), []
    for _ in range(max_new):
        logits = plain_forward(cfg, weights, tokens, compute)[-1]
        tok = plain_sample(logits.to(torch.float32), temperature, top_k, top_p, rng)
        if tok in stop:
            break
        out.append(tok)
        tokens.append(tok)
    return out
