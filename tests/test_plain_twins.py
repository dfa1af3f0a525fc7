"""The kernels' plain C++ twins against the plain PyTorch implementation (float64), on the CPU: two readings of
the same formulas, written apart, must agree to the rounding of the output type."""
import math

import pytest
import torch

from llm_rs_amd.kernels import EPI_ACCUM_F32, EPI_STORE, EPI_STORE_F32, EPI_SWIGLU, NextNorm, NormedRows
from plain_llama import (plain_attention, plain_inv_freq, plain_probabilities, plain_rmsnorm, plain_rope,
                         plain_silu)
from plain_twins import twins

DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(got, want, dtype, floor=1e-6):
    """Within a rounding of the output type (and a floor for sums that cancel)."""
    rel = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -22
    err = (got.double() - want.double()).abs()
    assert (err <= want.double().abs() * rel + floor).all(), float(err.max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_rows(dtype):
    table = rnd((37, 24), dtype, 1)
    tokens = torch.tensor([5, 0, 36, 5], dtype=torch.int32)
    out = torch.zeros((4, 24), dtype=torch.float32)
    twins().embed_rows(out, table, tokens, 1.5)
    assert torch.equal(out, (table[tokens.long()].double() * 1.5).float())
    with pytest.raises(ValueError):
        twins().embed_rows(out, table, torch.tensor([1, 2, 3, 37], dtype=torch.int32))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm(dtype):
    x, w = rnd((5, 100), torch.float32, 2, 3.0), rnd((100,), torch.float32, 3) * 0.1 + 1
    out = torch.zeros((5, 100), dtype=dtype)
    twins().rmsnorm(out, x, w, 1e-5)
    close(out, plain_rmsnorm(x.double(), w.double(), 1e-5), dtype)
    rows = torch.tensor([4, 1], dtype=torch.int32)
    part = torch.zeros((2, 100), dtype=dtype)
    twins().rmsnorm(part, x, w, 1e-5, rows)
    assert torch.equal(part, out[rows.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("epi", [EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU])
def test_gemm(dtype, epi):
    M, N, K = 7, 36, 50
    a, w = rnd((M, K + 3), dtype, 4)[:, :K], rnd((N, K), dtype, 5, 0.2)
    sums = a.double() @ w.double().T
    if epi == EPI_SWIGLU:
        out = torch.zeros((M, N // 2), dtype=dtype)
        want = plain_silu(sums[:, 0::2]) * sums[:, 1::2]
    elif epi == EPI_STORE:
        out, want = torch.zeros((M, N), dtype=dtype), sums
    else:
        out = rnd((M, N), torch.float32, 6) if epi == EPI_ACCUM_F32 else torch.zeros((M, N))
        want = sums + (out.double() if epi == EPI_ACCUM_F32 else 0)
    twins().gemm(a, w, out, epi)
    close(out, want, out.dtype, 1e-5)


def test_gemm_with_a_norm_left_to_it_and_one_left_for_the_next():
    M, N, K = 5, 40, 64
    h = rnd((M, K), torch.float32, 7, 2.0)
    nw = rnd((K,), torch.float32, 8) * 0.1 + 1
    y = (h * nw).bfloat16()
    sumsq = (h.double() ** 2).view(M, K // 16, 16).sum(-1).float()
    w = rnd((N, K), torch.bfloat16, 9, 0.1)
    out = torch.zeros((M, N), dtype=torch.bfloat16)
    twins().gemm(NormedRows(y, sumsq, 1e-5), w, out)
    inv = 1.0 / torch.sqrt((h.double() ** 2).mean(-1, keepdim=True) + 1e-5)
    close(out, (y.double() * inv) @ w.double().T, torch.bfloat16, 1e-4)
    # what a product leaves for the next norm: rows times weight and sums of squares, or the finished norm
    stream = rnd((M, N), torch.float32, 10)
    a = rnd((M, K), torch.bfloat16, 11)
    w2 = rnd((N, K), torch.bfloat16, 12, 0.1)
    nw2 = rnd((N,), torch.float32, 13) * 0.1 + 1
    new = stream.double() + a.double() @ w2.double().T
    left = NextNorm(torch.zeros((M, N), dtype=torch.bfloat16), torch.zeros((M, 3)), nw2)
    s1 = stream.clone()
    twins().gemm(a, w2, s1, EPI_ACCUM_F32, None, left)
    close(s1, new, torch.float32, 1e-5)
    close(left.y, s1.double() * nw2.double(), torch.bfloat16)
    padded = torch.zeros((M, 48), dtype=torch.float64)
    padded[:, :N] = s1.double()
    close(left.sumsq, (padded ** 2).view(M, 3, 16).sum(-1), torch.float32)
    whole = NextNorm(torch.zeros((M, N), dtype=torch.bfloat16), None, nw2, 1e-5)
    s2 = stream.clone()
    twins().gemm(a, w2, s2, EPI_ACCUM_F32, None, whole)
    assert torch.equal(s1, s2)
    close(whole.y, plain_rmsnorm(s2.double(), nw2.double(), 1e-5), torch.bfloat16)


def _cache(num_pages, n_kv, ps, hd, dtype):
    return torch.zeros((num_pages, n_kv, ps, hd), dtype=dtype), torch.zeros((num_pages, n_kv, hd, ps), dtype=dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interleaved,rot", [(False, 16), (True, 16), (False, 8), (True, 0)])
def test_rope_kv_write(dtype, interleaved, rot):
    T, H, KV, hd, ps, pages = 6, 4, 2, 16, 4, 5
    qkv = rnd((T, (H + 2 * KV) * hd), dtype, 14)
    before = qkv.clone()
    positions = torch.tensor([0, 1, 7, 300, 2, 9], dtype=torch.int32)
    slots = torch.tensor([3, 0, 19, 8, 5, 14], dtype=torch.int32)
    inv_freq = plain_inv_freq(rot, 10000.0, None) if rot else None
    kc, vc = _cache(pages, KV, ps, hd, dtype)
    twins().rope_kv_write(qkv, positions, slots, inv_freq, rot, interleaved, kc, vc, H, KV, hd, ps, pages, True)
    q = before[:, :H * hd].double().view(T, H, hd)
    k = before[:, H * hd:(H + KV) * hd].double().view(T, KV, hd)
    v = before[:, (H + KV) * hd:].double().view(T, KV, hd)
    if rot:
        layout = "interleaved" if interleaved else "split_half"
        q, k = plain_rope(q, positions, inv_freq, layout), plain_rope(k, positions, inv_freq, layout)
    close(qkv[:, :H * hd].view(T, H, hd), q, dtype)
    assert torch.equal(qkv[:, H * hd:], before[:, H * hd:]), "k and v stay as they are in qkv"
    for t in range(T):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        close(kc[page, :, off, :], k[t], dtype)
        close(vc[page, :, :, off], v[t], dtype)
    assert int((kc != 0).sum()) <= T * KV * hd, "nothing written elsewhere"


@pytest.mark.parametrize("dtype", DTYPES)
def test_qkv_rope_cache(dtype):
    T, H, KV, hd, ps, pages, K, rot = 5, 4, 2, 16, 4, 6, 48, 8
    x, w = rnd((T, K), dtype, 15), rnd(((H + 2 * KV) * hd, K), dtype, 16, 0.2)
    positions = torch.tensor([0, 3, 50, 1, 2], dtype=torch.int32)
    slots = torch.tensor([1, 23, 8, 4, 17], dtype=torch.int32)
    inv_freq = plain_inv_freq(rot, 10000.0, None)
    qkv = torch.zeros((T, (H + 2 * KV) * hd), dtype=dtype)
    kc, vc = _cache(pages, KV, ps, hd, dtype)
    twins().qkv_rope_cache(x, w, qkv, positions, slots, inv_freq, rot, kc, vc, H, KV, hd, ps, pages, True)
    full = x.double() @ w.double().T
    q = plain_rope(full[:, :H * hd].view(T, H, hd), positions, inv_freq, "interleaved")
    k = plain_rope(full[:, H * hd:(H + KV) * hd].view(T, KV, hd), positions, inv_freq, "interleaved")
    v = full[:, (H + KV) * hd:].view(T, KV, hd)
    close(qkv[:, :H * hd].view(T, H, hd), q, dtype, 1e-5)
    for t in range(T):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        close(kc[page, :, off, :], k[t], dtype, 1e-5)
        close(vc[page, :, :, off], v[t], dtype, 1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [0, 7])
def test_attention_over_pages(dtype, window):
    H, KV, hd, ps = 6, 2, 20, 4
    lens = [13, 5]
    g = torch.Generator().manual_seed(17)
    ks = [rnd((n, KV, hd), dtype, 20 + i) for i, n in enumerate(lens)]
    vs = [rnd((n, KV, hd), dtype, 30 + i) for i, n in enumerate(lens)]
    pages_per = [-(-n // ps) for n in lens]
    num_pages = sum(pages_per) + 2
    perm = torch.randperm(num_pages, generator=g)
    table = torch.zeros((2, max(pages_per)), dtype=torch.int32)
    kc, vc = _cache(num_pages, KV, ps, hd, dtype)
    at = 0
    for r, n in enumerate(lens):
        for i in range(pages_per[r]):
            page = int(perm[at]); at += 1
            table[r, i] = page
            lo, hi = i * ps, min((i + 1) * ps, n)
            kc[page, :, :hi - lo, :] = ks[r][lo:hi].permute(1, 0, 2)
            vc[page, :, :, :hi - lo] = vs[r][lo:hi].permute(1, 2, 0)
    # request 0: its last four tokens; request 1: its last token
    pos = [list(range(9, 13)), [4]]
    q = rnd((5, H * hd), dtype, 40)
    entry = torch.tensor([0, 0, 0, 0, 1], dtype=torch.int32)
    positions = torch.tensor(pos[0] + pos[1], dtype=torch.int32)
    out = torch.zeros((5, H * hd), dtype=dtype)
    twins().attention(q, out, kc, vc, table, entry, positions, None, None, H, KV, hd, ps, num_pages, window, 0.3)
    at = 0
    for r, p in enumerate(pos):
        n = lens[r]
        qq = torch.zeros((n, H, hd), dtype=torch.float64)
        for i, place in enumerate(p):
            qq[place] = q[at + i].double().view(H, hd)
        want = plain_attention(qq, ks[r].double(), vs[r].double(), 0.3, window)
        for i, place in enumerate(p):
            close(out[at + i].view(H, hd), want[place], dtype, 1e-6)
        at += len(p)


def test_argmax_and_sampling():
    V = 300
    logits = rnd((6, V), torch.float32, 50, 3.0)
    logits[1, [10, 20]] = 50.0          # equal maxima: the lower index
    out = torch.zeros(6, dtype=torch.int32)
    twins().argmax_rows(logits, out)
    assert out.tolist() == [int(logits[i].argmax()) if i != 1 else 10 for i in range(6)]
    settings = [(0.31, 0.8, 0, 1.0), (0.77, 0.7, 40, 0.9), (0.5, 1.3, 5, 1.0), (0.999, 0.5, 0, 0.8), (0.02, 1.0, 3, 0.95), (0.4, 0.0, 0, 1.0)]
    words = torch.zeros((6, 4), dtype=torch.int32)
    for i, (u, t, k, p) in enumerate(settings):
        f = torch.tensor([u, t, p], dtype=torch.float32).view(torch.int32)
        words[i, 0], words[i, 1], words[i, 2], words[i, 3] = f[0], f[1], k, f[2]
    probs = torch.zeros((6, V), dtype=torch.float64)
    twins().sample_rows(logits, words, out, probs)
    for i, (u, t, k, p) in enumerate(settings):
        if t == 0.0:
            assert int(out[i]) == int(logits[i].argmax())
            continue
        want = plain_probabilities(logits[i], t, k, p)
        assert float((probs[i] - want).abs().max()) < 1e-6 and torch.equal(probs[i] > 0, want > 0)
        cum = torch.cumsum(want, 0)
        tok = int(out[i])
        assert float(cum[tok] - want[tok]) - 1e-6 <= u < float(cum[tok]) + 1e-6


def test_cast_and_softcap():
    src = rnd((1000,), torch.float32, 60, 100.0)
    dst = torch.zeros(1000, dtype=torch.bfloat16)
    twins().cast(dst, src)
    assert torch.equal(dst, src.bfloat16())
    half = src.half()
    back = torch.zeros(1000, dtype=torch.float32)
    twins().cast(back, half)
    assert torch.equal(back, half.float())
    logits = rnd((3, 50), torch.float32, 61, 20.0)
    want = 30.0 * torch.tanh(logits.double() * 0.5 / 30.0)
    twins().scale_softcap_rows(logits, 0.5, 30.0)
    close(logits, want, torch.float32)
