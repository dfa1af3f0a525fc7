"""Each device kernel against its plain C++ twin: one call, the same arguments, made on the device and on the
host, and the outputs compared to the rounding of their type."""
import math

import pytest
import torch

from llm_rs_amd.kernels import (EPI_ACCUM_F32, EPI_STORE, EPI_STORE_F32, EPI_SWIGLU, NextNorm, NormedRows, kernels)
from plain_llama import plain_inv_freq
from plain_twins import twins

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def dev(x):
    if isinstance(x, torch.Tensor):
        return x.to(DEV)
    if isinstance(x, NormedRows):
        return NormedRows(x.y.to(DEV), x.sumsq.to(DEV), x.eps)
    if isinstance(x, NextNorm):
        return NextNorm(x.y.to(DEV), None if x.sumsq is None else x.sumsq.to(DEV), x.weight.to(DEV), x.eps)
    return x


def both(name, args, outs):
    """Calls kernel `name` on the device and its twin on the host with `args` (tensors given on the host; the device
    gets copies); returns [(device result, twin result)] for the positions `outs` of args (an int, or (int, attribute))."""
    on_dev = [dev(a) for a in args]
    getattr(kernels(), name)(*on_dev)
    torch.cuda.synchronize()
    getattr(twins(), name)(*args)
    pick = lambda seq, o: getattr(seq[o[0]], o[1]) if isinstance(o, tuple) else seq[o]
    return [(pick(on_dev, o).cpu(), pick(args, o)) for o in outs]


def close(pair, floor=1e-6, sums_of=0):
    """Within a rounding of the output type; sums of `sums_of` products in 32-bit may differ from the twin's (in
    double) by their own rounding as well."""
    got, want = pair
    rel = 2.0 ** -7 if got.dtype == torch.bfloat16 else 2.0 ** -21
    err = (got.double() - want.double()).abs()
    slack = floor + 1e-6 * math.sqrt(sums_of) * max(1.0, float(want.double().abs().max()))
    assert (err <= want.double().abs() * rel + slack).all(), float(err.max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [328, 35, 4096])
def test_embed_rows(dtype, D):
    table = rnd((1001, D), dtype, 1)
    tokens = torch.randint(0, 1001, (37,), generator=torch.Generator().manual_seed(2)).to(torch.int32)
    (pair,) = both("embed_rows", [torch.zeros((37, D)), table, tokens, 0.7], [0])
    assert torch.equal(*pair)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [328, 4096, 20000])
def test_rmsnorm(dtype, D):
    x, w = rnd((9, D), torch.float32, 3, 4.0), rnd((D,), torch.float32, 4) * 0.1 + 1
    rows = torch.tensor([8, 0, 3], dtype=torch.int32)
    close(both("rmsnorm", [torch.zeros((9, D), dtype=dtype), x, w, 1e-5], [0])[0])
    close(both("rmsnorm", [torch.zeros((3, D), dtype=dtype), x, w, 2e-6, rows], [0])[0])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("epi", [EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU])
@pytest.mark.parametrize("M,N,K", [(1, 520, 328), (8, 1024, 512), (50, 600, 264), (300, 512, 448)])
def test_gemm(dtype, epi, M, N, K):
    a, w = rnd((M, K), dtype, 5), rnd((N, K), dtype, 6, 0.1)
    if epi == EPI_SWIGLU:
        out = torch.zeros((M, N // 2), dtype=dtype)
    elif epi == EPI_STORE:
        out = torch.zeros((M, N), dtype=dtype)
    else:
        out = rnd((M, N), torch.float32, 7)
    k = kernels()
    n = k.gemm_workspace_floats(M, N, K)
    on_dev = [a.to(DEV), w.to(DEV), out.to(DEV), epi, torch.empty(n, dtype=torch.float32, device=DEV) if n else None]
    k.gemm(*on_dev)
    twins().gemm(a, w, out, epi)
    close((on_dev[2].cpu(), out), 1e-5, sums_of=K if dtype == torch.float32 else 0)


@pytest.mark.parametrize("M,N,K", [(4, 1024, 512), (16, 600, 256)])
def test_gemm_norm_left_to_it_and_left_for_the_next(M, N, K):
    h = rnd((M, K), torch.float32, 8, 2.0)
    nw = rnd((K,), torch.float32, 9) * 0.1 + 1
    rows = NormedRows((h * nw).bfloat16(), (h.double() ** 2).view(M, K // 16, 16).sum(-1).float(), 1e-5)
    w = rnd((N, K), torch.bfloat16, 10, 0.1)
    close(both("gemm", [rows, w, torch.zeros((M, N), dtype=torch.bfloat16)], [2])[0], 1e-4)
    nw2 = rnd((N,), torch.float32, 11) * 0.1 + 1
    left = NextNorm(torch.zeros((M, N), dtype=torch.bfloat16), torch.zeros((M, -(-N // 16))), nw2)
    a = rnd((M, K), torch.bfloat16, 12)
    stream, y, sumsq = both("gemm", [a, w, rnd((M, N), torch.float32, 13), EPI_ACCUM_F32, None, left], [2, (5, "y"), (5, "sumsq")])
    close(stream, 1e-5)
    close(y, 1e-5)
    close(sumsq, 1e-5)


def test_gemm_finishes_the_next_norm():
    M, N, K = 40, 1024, 2048
    k = kernels()
    assert k.gemm_norms_whole(M, N, K)
    a, w = rnd((M, K), torch.bfloat16, 14), rnd((N, K), torch.bfloat16, 15, 0.1)
    nw = rnd((N,), torch.float32, 16) * 0.1 + 1
    stream = rnd((M, N), torch.float32, 17)
    y = torch.zeros((M, N), dtype=torch.bfloat16)
    ws = torch.empty(k.gemm_workspace_floats(M, N, K), dtype=torch.float32, device=DEV)
    d_stream, d_y = stream.to(DEV), y.to(DEV)
    k.gemm(a.to(DEV), w.to(DEV), d_stream, EPI_ACCUM_F32, ws, NextNorm(d_y, None, nw.to(DEV), 1e-5))
    twins().gemm(a, w, stream, EPI_ACCUM_F32, None, NextNorm(y, None, nw, 1e-5))
    close((d_stream.cpu(), stream), 1e-5)
    close((d_y.cpu(), y), 1e-5)


def _cache(num_pages, n_kv, ps, hd, dtype):
    return torch.zeros((num_pages, n_kv, ps, hd), dtype=dtype), torch.zeros((num_pages, n_kv, hd, ps), dtype=dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interleaved,rot,T", [(False, 64, 9), (True, 64, 40), (False, 32, 3), (True, 0, 5)])
def test_rope_kv_write(dtype, interleaved, rot, T):
    H, KV, hd, ps, pages = 6, 2, 64, 16, 7
    qkv = rnd((T, (H + 2 * KV) * hd), dtype, 18)
    g = torch.Generator().manual_seed(19)
    positions = torch.randint(0, 3000, (T,), generator=g).to(torch.int32)
    slots = torch.randperm(pages * ps, generator=g)[:T].to(torch.int32)
    inv_freq = plain_inv_freq(rot, 500000.0, None) if rot else None
    kc, vc = _cache(pages, KV, ps, hd, dtype)
    q, k, v = both("rope_kv_write", [qkv, positions, slots, inv_freq, rot, interleaved, kc, vc, H, KV, hd, ps, pages, True], [0, 6, 7])
    # an angle of thousands of radians, taken in 32-bit: its sine and cosine carry that angle's rounding on both sides alike
    close(q, 2e-6)
    close(k, 2e-6)
    assert torch.equal(*v)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [1, 8, 40, 100])
def test_qkv_rope_cache(dtype, T):
    H, KV, hd, ps, pages, K, rot = 8, 2, 64, 16, 9, 512, 64
    x, w = rnd((T, K), dtype, 20), rnd(((H + 2 * KV) * hd, K), dtype, 21, 0.1)
    g = torch.Generator().manual_seed(22)
    positions = torch.randint(0, 2000, (T,), generator=g).to(torch.int32)
    slots = torch.randperm(pages * ps, generator=g)[:T].to(torch.int32)
    inv_freq = plain_inv_freq(rot, 10000.0, None)
    kc, vc = _cache(pages, KV, ps, hd, dtype)
    qkv = torch.zeros((T, (H + 2 * KV) * hd), dtype=dtype)
    q, k, v = both("qkv_rope_cache", [x, w, qkv, positions, slots, inv_freq, rot, kc, vc, H, KV, hd, ps, pages, True], [2, 7, 8])
    sums = K if dtype == torch.float32 else 0
    # more than 64 tokens: the product and the rotation are two kernels, and the sums are rounded between them: a
    # rotated value carries the roundings of both values of its pair, which may be far larger than itself
    floor = 1e-5 + (2.0 ** -8 * float(q[1].double().abs().max()) if T > 64 and dtype == torch.bfloat16 else 0.0)
    close((q[0][:, :H * hd], q[1][:, :H * hd]), floor, sums)
    close(k, floor, sums)
    close(v, 1e-5, sums)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,ps,window", [(8, 2, 128, 16, 0), (8, 2, 128, 16, 100), (6, 3, 48, 8, 0), (4, 4, 20, 4, 30), (16, 2, 64, 16, 0)])
def test_attention(dtype, H, KV, hd, ps, window):
    """Three requests: a prompt portion, a whole short prompt and a decoding one, over scattered pages."""
    lens = [300, 17, 650]
    g = torch.Generator().manual_seed(hd + window)
    pages_per = [-(-n // ps) for n in lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g)
    table = torch.zeros((3, max(pages_per)), dtype=torch.int32)
    kc, vc = _cache(num_pages, KV, ps, hd, dtype)
    at = 0
    for r, n in enumerate(lens):
        for i in range(pages_per[r]):
            page = int(perm[at]); at += 1
            table[r, i] = page
            fill = min(ps, n - i * ps)
            kc[page, :, :fill, :] = rnd((KV, fill, hd), dtype, 100 * r + i)
            vc[page, :, :, :fill] = rnd((KV, hd, fill), dtype, 5000 + 100 * r + i)
    pos = [list(range(250, 300)), list(range(17)), [649]]
    counts = [len(p) for p in pos]
    T = sum(counts)
    q = rnd((T, H * hd), dtype, 23)
    entry = torch.cat([torch.full((c,), r, dtype=torch.int32) for r, c in enumerate(counts)])
    positions = torch.tensor([p for ps_ in pos for p in ps_], dtype=torch.int32)
    q_starts = torch.tensor([0, 50, 67, 68], dtype=torch.int32)
    seq_lens = torch.tensor(lens, dtype=torch.int32)
    scratch = torch.empty(kernels().attention_scratch_floats(3, H, hd, 650, KV, 1), dtype=torch.float32)
    args = [q, torch.zeros((T, H * hd), dtype=dtype), kc, vc, table, entry, positions, q_starts, seq_lens, H, KV, hd, ps,
            num_pages, window, 1.0 / math.sqrt(hd), scratch, 650, 1]
    (pair,) = both("attention", args, [1])
    got, want = pair
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5        # (bfloat16: the probabilities are rounded for the second product)
    assert float((got.double() - want.double()).abs().max()) <= tol


def test_argmax_and_sample_rows():
    V = 5003
    logits = rnd((12, V), torch.float32, 24, 3.0)
    logits[1, [700, 4000]] = 60.0
    (pair,) = both("argmax_rows", [logits, torch.zeros(12, dtype=torch.int32)], [1])
    assert torch.equal(*pair) and int(pair[0][1]) == 700
    g = torch.Generator().manual_seed(25)
    settings = [(0.8, 0, 1.0), (0.7, 40, 0.9), (1.3, 5, 1.0), (0.5, 0, 0.8), (1.0, 2000, 0.95), (0.0, 0, 1.0)] * 2
    words = torch.zeros((12, 4), dtype=torch.int32)
    us = []
    for i, (t, kk, p) in enumerate(settings):
        u = float(torch.rand(1, generator=g))
        us.append(u)
        f = torch.tensor([u, t, p], dtype=torch.float32).view(torch.int32)
        words[i, 0], words[i, 1], words[i, 2], words[i, 3] = f[0], f[1], kk, f[2]
    out = torch.zeros(12, dtype=torch.int32, device=DEV)
    kernels().sample_rows(logits.to(DEV), words.to(DEV), out)
    probs = torch.zeros((12, V), dtype=torch.float64)
    twin_out = torch.zeros(12, dtype=torch.int32)
    twins().sample_rows(logits, words, twin_out, probs)
    cum = torch.cumsum(probs, 1)
    for i, tok in enumerate(out.tolist()):
        # the device sums in 32-bit: a uniform within 1e-5 of an interval's edge may fall to either side
        assert probs[i, tok] > 0 and float(cum[i, tok] - probs[i, tok]) - 1e-5 <= us[i] < float(cum[i, tok]) + 1e-5
        if abs(float(cum[i, twin_out[i]]) - us[i]) > 1e-4 and abs(float(cum[i, twin_out[i]] - probs[i, twin_out[i]]) - us[i]) > 1e-4:
            assert tok == int(twin_out[i])


def test_place_ids():
    """Sampled ids into the next step's tokens: pairs out of range and ids outside the vocabulary change nothing."""
    g = torch.Generator().manual_seed(31)
    tokens = torch.randint(0, 900, (700,), generator=g).to(torch.int32)
    ids = torch.randint(0, 900, (300,), generator=g).to(torch.int32)
    ids[7], ids[8] = -3, 900                                        # not in a vocabulary of 900
    rows = torch.randperm(700, generator=g)[:300].to(torch.int32)
    sources = torch.randperm(300, generator=g).to(torch.int32)
    rows[5], rows[6], sources[9], sources[10] = -1, 700, -1, 300    # outside either array
    (pair,) = both("place_ids", [tokens.clone(), rows, sources, ids, 900], [0])
    assert torch.equal(*pair)
    got = pair[0]
    changed = 0
    for i in range(300):
        r, s_ = int(rows[i]), int(sources[i])
        if 0 <= r < 700 and 0 <= s_ < 300 and 0 <= int(ids[s_]) < 900:
            assert int(got[r]) == int(ids[s_]); changed += 1
    untouched = torch.ones(700, dtype=torch.bool)
    untouched[rows[(rows >= 0) & (rows < 700)].long()] = False
    assert torch.equal(got[untouched], tokens[untouched]) and changed >= 290


def test_cast_and_softcap():
    src = rnd((100003,), torch.float32, 26, 50.0)
    assert torch.equal(*both("cast", [torch.zeros(100003, dtype=torch.bfloat16), src], [0])[0])
    assert torch.equal(*both("cast", [torch.zeros(100003, dtype=torch.float32), src.half()], [0])[0])
    assert torch.equal(*both("cast", [torch.zeros(100003, dtype=torch.bfloat16), src.half()], [0])[0])
    close(both("scale_softcap_rows", [rnd((5, 1000), torch.float32, 27, 20.0), 0.5, 30.0], [0])[0])
    close(both("scale_softcap_rows", [rnd((5, 1000), torch.float32, 28, 20.0), 2.0, 0.0], [0])[0])
