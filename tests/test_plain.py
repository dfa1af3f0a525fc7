"""What fixes the plain implementation beside the reference's text: special cases
that reduce to a library routine, invariants, and the reference's own constants;
each chosen so that a plausible mistake (a wrong sign or pairing, a norm in the
wrong place, a scale before the dot's sum) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from plain_llama import (PlainXorshift, plain_argmax, plain_attention, plain_forward, plain_inv_freq,
                         plain_probabilities, plain_rmsnorm, plain_rope, plain_sample, plain_silu, plain_swiglu)
from llm_rs_amd import LlamaConfig, random_model_tensors
from tiny_configs import TINY_A, TINY_B

torch.manual_seed(0)
D = torch.float64


def test_rmsnorm_is_the_library_routine_and_scale_free():
    x, w = torch.randn(5, 48, dtype=D), torch.randn(48, dtype=D)
    assert torch.allclose(plain_rmsnorm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), atol=1e-12)
    y = plain_rmsnorm(x, torch.ones(48, dtype=D), 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=D), atol=1e-9)              # unit RMS
    assert torch.allclose(plain_rmsnorm(7.0 * x, w, 1e-14), plain_rmsnorm(x, w, 1e-14), atol=1e-9)
    assert not torch.allclose(plain_rmsnorm(x, w, 1e-5), plain_rmsnorm(x, 1 + w, 1e-5))      # no (1 + w)
    big_eps = plain_rmsnorm(x, w, 10.0)
    assert (big_eps.abs() < plain_rmsnorm(x, w, 1e-5).abs()).all()                          # eps sits under the root, added to the mean


def test_rope_is_a_complex_rotation():
    T, H, d = 6, 3, 16
    x = torch.randn(T, H, d, dtype=D)
    pos = torch.tensor([0, 1, 2, 10, 11, 300])
    inv = plain_inv_freq(d, 10000.0, None)
    assert torch.allclose(inv.double(), 1.0 / 10000.0 ** (torch.arange(0, d, 2, dtype=D) / d), rtol=1e-6)
    y = plain_rope(x, pos, inv)
    angle = (pos.float()[:, None] * inv[None, :]).double()
    z = torch.complex(x[..., :d // 2], x[..., d // 2:]) * torch.polar(torch.ones_like(angle), angle)[:, None, :]
    assert torch.allclose(y[..., :d // 2], z.real, atol=1e-12) and torch.allclose(y[..., d // 2:], z.imag, atol=1e-12)
    assert torch.equal(y[0], x[0]), "position 0 is the identity"
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-12)
    # interleaved is split-half under the fixed permutation of features
    perm = torch.cat([torch.arange(0, d, 2), torch.arange(1, d, 2)])
    yi = plain_rope(x, pos, inv, "interleaved")
    assert torch.allclose(yi[..., perm], plain_rope(x[..., perm], pos, inv, "split_half"), atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    d = 32
    q, k = torch.randn(1, 1, d, dtype=D), torch.randn(1, 1, d, dtype=D)
    inv = plain_inv_freq(d, 500000.0, TINY_B["rope_scaling"])
    def score(m, n):
        return float((plain_rope(q, torch.tensor([m]), inv) * plain_rope(k, torch.tensor([n]), inv)).sum())
    assert abs(score(7, 3) - score(107, 103)) < 1e-4 and abs(score(7, 3) - score(3, 7)) > 1e-3


def test_llama3_scaling_bands():
    d, theta = 64, 500000.0
    plain = plain_inv_freq(d, theta, None).double()
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    scaled = plain_inv_freq(d, theta, sc).double()
    assert torch.allclose(plain_inv_freq(d, theta, {**sc, "factor": 1.0}).double(), plain, rtol=1e-6)
    wavelength = 2 * math.pi / plain
    high, low = wavelength < 64 / 4.0, wavelength > 64 / 1.0
    assert high.any() and low.any() and (~high & ~low).any(), "the case must have all three bands"
    assert torch.allclose(scaled[high], plain[high], rtol=1e-6), "short wavelengths keep their frequency"
    assert torch.allclose(scaled[low], plain[low] / 8.0, rtol=1e-6), "long wavelengths are stretched by the factor"
    mid = scaled[~high & ~low] / plain[~high & ~low]
    assert ((mid > 1 / 8.0) & (mid < 1.0)).all() and (mid[:-1] >= mid[1:]).all(), "the band between blends monotonically"


def test_llama3_scaling_blends_in_frequency_not_in_wavelength():
    """Between the two band edges the new frequency is a straight line in L / wavelength (that is,
    in the frequency itself) from freq / factor at the low edge to freq at the high edge.  A
    frequency placed a quarter, a half and three quarters of the way between the edges must come out
    scaled by (1 - s) / factor + s for s = 1/4, 1/2, 3/4 (0.344, 0.563, 0.781 with factor 8); blending along
    the wavelength instead gives 0.160, 0.222, 0.364, and a line that runs the other way 0.781, 0.563, 0.344.
    The same through the engine's own table (parts/rope.py), which the kernels multiply positions by."""
    from llm_rs_amd.parts import rope_inv_freq
    L, factor, low, high = 64.0, 8.0, 1.0, 4.0
    sc = dict(rope_type="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high, original_max_position_embeddings=int(L))
    for s_want in (0.25, 0.5, 0.75):
        turns = low + s_want * (high - low)             # L / wavelength of the frequency under test
        freq = 2 * math.pi * turns / L
        theta = freq ** -2.0                            # rotary_dim 4: pair 1 has frequency theta^(-1/2)
        want = freq * ((1 - s_want) / factor + s_want)
        got = float(plain_inv_freq(4, theta, sc)[1])
        assert abs(got / want - 1) < 1e-6, (s_want, got / freq)
        assert abs(float(rope_inv_freq(4, theta, sc)[1]) / want - 1) < 1e-6
        in_wavelength = 1.0 / ((1 - s_want) * factor + s_want)      # what a blend along the wavelength would give
        assert abs(got / freq - in_wavelength) > 0.05
    # the edges themselves: kept at the high edge, divided by the factor at the low edge, no jump next to them
    for turns, ratio in ((high * 1.0001, 1.0), (high * 0.9999, 1.0), (low * 1.0001, 1 / factor), (low * 0.9999, 1 / factor)):
        freq = 2 * math.pi * turns / L
        assert abs(float(plain_inv_freq(4, freq ** -2.0, sc)[1]) / freq - ratio) < 2e-4


def test_attention_special_cases():
    T, H, d = 9, 4, 8
    q, k, v = (torch.randn(T, H, d, dtype=D) for _ in range(3))
    # plain multi-head attention = the library routine with a causal mask
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(plain_attention(q, k, v), lib, atol=1e-12)
    assert torch.allclose(plain_attention(q, k, v)[0], v[0], atol=1e-12), "the first query sees one key"
    # equal keys: the mean of the values over the causal prefix
    same = plain_attention(q, k[:1].expand(T, H, d), v)
    assert torch.allclose(same, torch.cumsum(v, 0) / torch.arange(1, T + 1, dtype=D)[:, None, None], atol=1e-12)
    # grouped queries: head h reads kv head h // (H / KV)
    kg, vg = torch.randn(T, 2, d, dtype=D), torch.randn(T, 2, d, dtype=D)
    assert torch.allclose(plain_attention(q, kg, vg),
                          plain_attention(q, kg.repeat_interleave(2, 1), vg.repeat_interleave(2, 1)), atol=1e-12)
    # later tokens do not change earlier rows
    k2, v2 = k.clone(), v.clone()
    k2[5:], v2[5:] = torch.randn(4, H, d, dtype=D), torch.randn(4, H, d, dtype=D)
    assert torch.allclose(plain_attention(q, k2, v2)[:5], plain_attention(q, k, v)[:5], atol=1e-12)
    # a window of w keys: w = 1 returns the token's own value
    assert torch.allclose(plain_attention(q, k, v, window=1), v, atol=1e-12)
    assert torch.allclose(plain_attention(q, k, v, window=T), plain_attention(q, k, v), atol=1e-12)


def test_swiglu():
    x = torch.randn(4, 6, dtype=D)
    assert torch.allclose(plain_silu(x), F.silu(x), atol=1e-12)
    wg, wu, wd = torch.randn(10, 6, dtype=D), torch.randn(10, 6, dtype=D), torch.randn(6, 10, dtype=D)
    assert torch.allclose(plain_swiglu(x, wg, wu, wd), (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T, atol=1e-12)
    assert not torch.allclose(plain_swiglu(x, wg, wu, wd), plain_swiglu(x, wu, wg, wd)), "gate and up are not interchangeable"


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_forward_invariants(cfg):
    weights = random_model_tensors(LlamaConfig.from_dict(cfg), 0)
    toks = torch.randint(0, cfg["vocab_size"], (12,)).tolist()
    full = plain_forward(cfg, weights, toks)
    assert full.shape == (12, cfg["vocab_size"])
    assert torch.allclose(plain_forward(cfg, weights, toks[:7]), full[:7], atol=1e-10), "causal: a prefix gives the same rows"
    # only distances between positions count
    assert torch.allclose(plain_forward(cfg, weights, toks, position_offset=40), full, atol=1e-4)
    other = list(toks); other[3] = (other[3] + 1) % cfg["vocab_size"]
    changed = plain_forward(cfg, weights, other)
    assert torch.allclose(changed[:3], full[:3], atol=1e-10) and not torch.allclose(changed[3:], full[3:], atol=1e-6)
    if cfg["tie_word_embeddings"]:
        assert "lm_head.weight" not in weights


def test_sampling_rules():
    logits = torch.tensor([0.1, 2.0, 2.0, -1.0, 0.5])
    assert plain_argmax(logits) == 1, "lowest index among equal maxima"
    p = plain_probabilities(logits, 1.0, 0, 1.0)
    assert torch.allclose(p, torch.softmax(logits.double(), 0))
    assert torch.allclose(plain_probabilities(logits, 0.5, 0, 1.0), torch.softmax(logits.double() / 0.5, 0))
    p2 = plain_probabilities(logits, 1.0, 2, 1.0)
    assert p2.nonzero().flatten().tolist() == [1, 2] and abs(float(p2.sum()) - 1) < 1e-12
    p3 = plain_probabilities(logits, 1.0, 0, 0.5)          # 0.37 + 0.37 >= 0.5: two tokens
    assert p3.nonzero().flatten().tolist() == [1, 2]
    assert plain_probabilities(logits, 1.0, 0, 0.3).nonzero().flatten().tolist() == [1]
    rng = PlainXorshift(42)
    draws = [plain_sample(logits, 1.0, 0, 1.0, rng) for _ in range(3000)]
    freq = torch.bincount(torch.tensor(draws), minlength=5).double() / 3000
    assert (freq - p).abs().max() < 0.03
    assert all(plain_sample(logits, 1e-4, 0, 1.0, PlainXorshift(s)) in (1, 2) for s in range(5)), "T -> 0 is greedy"
    assert all(plain_sample(logits, 1.0, 1, 1.0, PlainXorshift(s)) == 1 for s in range(5)), "top_k = 1 is greedy"


def test_xorshift_constants():
    g = PlainXorshift(0)
    assert g.state == 0xDEADBEEFCAFE                      # src/sampler/mod.rs:10
    g = PlainXorshift(1)
    assert g.next_u64() == 1082269761 and 0.0 <= g.next_f32() < 1.0   # 1 ^ 1<<13 -> ^ >>7 -> ^ <<17


# Figures that were not made by this repository's code.  A reviewer computed them in float64 with an independent
# implementation of the Llama decoder (files in the HF layout: split-half rotation pairs, llama3 frequency scaling)
# from the tensors `random_model_tensors(cfg, 3)` and the tokens [(7 i + 3) mod vocab for i < 40], and handed over
# the numbers alone.  They pin the two things the reference's own files do not contain: the pairing of rotation
# under HF tensor names (the reference runs files converted to neighbouring pairs, src/arch/llama.rs:156,
# src/tensor/mod.rs:133-139) and the llama3 scaling of the frequencies (the reference scales nothing,
# shaders/ops.metal:1030).  Rotating neighbouring pairs on these files, or blending along the wavelength, fails them.
OUTSIDE_LOGITS = {
    "A": (TINY_A, {0: 0.101146, 1: -0.197046, 2: 0.007545, 128: -0.116913, 255: -0.016560}, 20, 109),
    "B": (TINY_B, {0: -0.182026, 1: 0.096695, 2: -0.054555, 192: -0.153350, 383: -0.267057}, 123, 325),
}
OUTSIDE_INV_FREQ = [     # (rotary width, factor, original length) -> {pair: frequency}; theta 5e5, low 1, high 4
    (32, 8.0, 64, {4: 0.004700753837823868, 8: 0.00017677668074611574, 12: 6.647869668086059e-06, 15: 5.677088097399974e-07}),
    (128, 8.0, 8192, {16: 0.03760603070259094, 32: 0.0005248460220173001, 48: 6.647869668086059e-06, 63: 3.068925877869333e-07}),
    (64, 32.0, 8192, {16: 0.000429556705057621, 24: 1.6619674170215148e-06, 31: 9.418306490260875e-08}),
]


@pytest.mark.parametrize("which", ["A", "B"])
def test_logits_computed_outside_this_repository(which):
    cfg, last_row, last_argmax, first_argmax = OUTSIDE_LOGITS[which]
    weights = random_model_tensors(LlamaConfig.from_dict(cfg), 3)
    tokens = [(7 * i + 3) % cfg["vocab_size"] for i in range(40)]
    logits = plain_forward(cfg, weights, tokens)
    for i, want in last_row.items():
        assert abs(float(logits[-1, i]) - want) < 2e-6, (i, float(logits[-1, i]), want)
    assert int(logits[-1].argmax()) == last_argmax and int(logits[0].argmax()) == first_argmax
    # the mistakes these figures are there to catch do move them
    wrong = plain_forward(cfg, weights, tokens, layout="interleaved")
    assert max(abs(float(wrong[-1, i]) - want) for i, want in last_row.items()) > 1e-4


@pytest.mark.parametrize("width,factor,length,want", OUTSIDE_INV_FREQ)
def test_llama3_frequencies_computed_outside_this_repository(width, factor, length, want):
    from llm_rs_amd.parts import rope_inv_freq
    sc = dict(rope_type="llama3", factor=factor, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=length)
    for table in (plain_inv_freq(width, 5e5, sc), rope_inv_freq(width, 5e5, sc)):
        for i, f in want.items():
            assert abs(float(table[i]) / f - 1) < 1e-6, (i, float(table[i]), f)
