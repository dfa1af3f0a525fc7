"""Each kernel alone against the plain reference of its part, at sizes other than
the tiny models': widths and vocabularies that are no power of two, head sizes in
steps of 16, any number of heads and groups."""
import math

import pytest
import torch

from llm_rs_amd.kernels import EPI_ACCUM_F32, EPI_STORE, EPI_STORE_F32, EPI_SWIGLU, KernelError, kernels
from plain_llama import plain_attention, plain_inv_freq, plain_rmsnorm, plain_rope, plain_silu

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


def out_tol(ref, dtype, floor):
    """Allowed error per element: half an ulp of the output type and then some, or a floor
    for sums that cancel (tests/ops.rs:142-145 uses |e|/64 and a floor for bfloat16 output)."""
    rel = 1.0 / 64 if dtype == torch.bfloat16 else 1e-5
    return ref.abs() * rel + floor


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_rows(dtype):
    table = rnd((1000, 200), dtype, 0)
    tokens = torch.tensor([0, 999, 17, 17, 500], dtype=torch.int32, device=DEV)
    out = torch.empty((5, 200), dtype=torch.float32, device=DEV)
    kernels().embed_rows(out, table, tokens)
    assert torch.equal(out, table[tokens.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,eps", [(200, 1e-5), (4104, 1e-6), (64, 1e-2), (4098, 1e-5), (20000, 1e-5)])
def test_rmsnorm(dtype, D, eps):
    x = rnd((9, D), torch.float32, 1, 3.0)
    w = rnd((D,), torch.float32, 2) * 0.1 + 1
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32, device=DEV)
    for r in (None, rows):
        n = 9 if r is None else 4
        out = torch.empty((n, D), dtype=dtype, device=DEV)
        kernels().rmsnorm(out, x, w, eps, r)
        src = x if r is None else x[r.long()]
        ref = plain_rmsnorm(src.double().cpu(), w.double().cpu(), eps)
        err = (out.double().cpu() - ref).abs()
        assert (err <= out_tol(ref, dtype, 1e-6)).all(), float(err.max())


GEMM_SHAPES = [(1, 40, 72), (5, 100, 200), (16, 48, 64), (17, 96, 320), (64, 256, 128), (65, 130, 1024),
               (130, 96, 320), (300, 520, 776), (257, 384, 96), (8, 1000, 4096), (33, 64, 20),
               (64, 200, 2048), (40, 1000, 1096), (64, 4096, 4096), (24, 520, 2048), (50, 64, 8200),
               (8, 38, 100), (3, 130, 4099), (1, 6, 20),
               # a few rows beyond whole 128-row tiles that would cost another round of the device (or the split of k): the few-row kernel takes them
               (2049, 4096, 2048), (1025, 4096, 4096), (2088, 4096, 2048),
               # 33 to 48 rows: blocks of three row tiles, in each of the few-row kernel's shapes
               (48, 4096, 4096), (36, 16400, 264), (47, 6144, 2048), (34, 2048, 2048), (41, 300, 136),
               # 256 x 192 tiles where they make whole rounds of the device and square ones do not; the last tile cut by N
               (2048, 6144, 128), (2048, 6100, 192), (1800, 6144, 64),
               # a round and a half of 16-feature blocks: blocks of 24 features (a tile and a half), the last one cut by N
               (8, 6144, 4096), (1, 6144, 2048), (16, 5120, 2048), (3, 6000, 4096), (5, 6152, 2048),
               (24, 6144, 2048), (64, 6144, 2048), (40, 6000, 2048), (30, 5128, 2048),
               (130, 200, 320), (300, 520, 768), (1000, 260, 1024), (65, 48, 64), (513, 1030, 128),
               # many features: blocks of several feature tiles that start their walk along k at staggered places
               (1, 16400, 200), (8, 16500, 328), (30, 17000, 136), (64, 16390, 264), (8, 28672, 256), (40, 28672, 192),
               # more large tiles than compute units, the last round not full: the features are split between two tile sizes
               (513, 25600, 64),
               # square large tiles of four waves (whole rounds; the last tile cut by M and N), and a width whose 16-bit
               # rows are no whole 16-byte pieces, which the eight-wave tiles take
               (2048, 8192, 512), (300, 41000, 192), (260, 41004, 128),
               # few tiles and a long k: the k range is split over blocks and the parts are added by a second kernel
               (100, 300, 4096), (257, 384, 1536), (200, 2048, 2048),
               # up to 256 rows and no more tiles than compute units: one block of eight waves per unit, four k-tiles in LDS
               (96, 6144, 2048), (256, 4096, 4096), (128, 28672, 1024), (192, 4100, 512),
               # a few rows beyond whole large tiles: those rows go to the kernel for few rows
               (1040, 10240, 128), (1080, 10500, 192), (2600, 4096, 1024),
               # long rows: narrow weights walk along k from staggered places too, with two feature tiles to a block
               (8, 300, 8256), (20, 8200, 16384), (3, 8200, 16400), (40, 520, 8192),
               # 17..64 rows on a weight of middling width: large tiles with the k range split over blocks
               (50, 4160, 1024), (64, 6144, 4096), (40, 5000, 2048), (33, 8192, 8192), (20, 6144, 4096),
               # 17..32 rows on a weight with few features: blocks of 64 features with the k range split over blocks
               (32, 4096, 4096), (20, 1000, 8200), (17, 2050, 2048)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("epi", [EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU])
def test_gemm(dtype, M, N, K, epi):
    pad = 24
    a_full = rnd((M, K + pad), dtype, 3)
    a = a_full[:, :K]                       # rows with a stride, as q inside qkv has
    w = rnd((N, K), dtype, 4, 0.1)
    acc = a.double().cpu() @ w.double().cpu().T
    floor = 2e-6 * math.sqrt(K) if dtype == torch.float32 else 1e-5 * math.sqrt(K)
    if epi == EPI_STORE:
        out = torch.zeros((M, N), dtype=dtype, device=DEV)
        ref, odt = acc, dtype
    elif epi == EPI_STORE_F32:
        out = torch.zeros((M, N), dtype=torch.float32, device=DEV)
        ref, odt = acc, torch.float32
    elif epi == EPI_ACCUM_F32:
        out = rnd((M, N), torch.float32, 5)
        ref, odt = out.double().cpu() + acc, torch.float32
    else:
        out = torch.zeros((M, N // 2), dtype=dtype, device=DEV)
        ref, odt = plain_silu(acc[:, 0::2]) * acc[:, 1::2], dtype
        floor *= 1 + 0.1 * math.sqrt(K)      # a sum's rounding error is multiplied by the other factor, of size 0.1 sqrt(K)
    n_ws = kernels().gemm_workspace_floats(M, N, K)
    ws = torch.empty(n_ws, dtype=torch.float32, device=DEV) if n_ws and dtype == torch.bfloat16 else None
    kernels().gemm(a, w, out, epi, ws)
    err = (out.double().cpu() - ref).abs()
    tol = out_tol(ref, odt, floor)
    assert (err <= tol).all(), f"max err {float(err.max())} at {int(err.argmax())}, tol there {float(tol.flatten()[err.argmax()])}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_rows_do_not_depend_on_batch(dtype):
    """Row t of the result depends on row t of the input only: the same row alone, in a
    small batch and in a large one agrees to rounding of the output."""
    K, N = 320, 200
    a = rnd((150, K), dtype, 6)
    w = rnd((N, K), dtype, 7, 0.1)
    outs = []
    for rows in ([7], list(range(4, 12)), list(range(150))):
        sub = a[rows].contiguous()
        out = torch.zeros((len(rows), N), dtype=torch.float32, device=DEV)
        kernels().gemm(sub, w, out, EPI_STORE_F32)
        outs.append(out[rows.index(7)].cpu())
    assert (outs[0] - outs[1]).abs().max() <= 2e-5 and (outs[0] - outs[2]).abs().max() <= 2e-5


@pytest.mark.parametrize("N,K", [(200, 320), (1000, 4096), (16500, 328), (28672, 256), (500, 8192), (8200, 16448)])
def test_gemm_small_batches_sum_in_one_order(N, K):
    """Up to 16 rows the matrix-core kernels add a feature's k-blocks in an order that the
    weight's shape fixes: a row's result is the same bits alone, among 8 or 16 rows.
    (With more rows a weight with few features has its k-blocks shared out over several
    blocks, and from 65 rows on the tiles are others: equal to rounding only.)"""
    a = rnd((32, K), torch.bfloat16, 16)
    w = rnd((N, K), torch.bfloat16, 17, 0.1)
    outs = []
    for rows in ([7], list(range(4, 12)), list(range(13)), list(range(16))):
        sub = a[rows].contiguous()
        out = torch.zeros((len(rows), N), dtype=torch.float32, device=DEV)
        ws = torch.empty(max(1, kernels().gemm_workspace_floats(len(rows), N, K)), dtype=torch.float32, device=DEV)
        kernels().gemm(sub, w, out, EPI_STORE_F32, ws)
        outs.append(out[rows.index(7)].cpu())
    for o in outs[1:]:
        assert torch.equal(outs[0], o)


def _rope_case(dtype, n_heads, n_kv, hd, rot, layout, page_size, theta=10000.0, scaling=None, repeat=1):
    """`repeat` > 1: more tokens, for the kernel that takes a token per block (16 tokens and more)."""
    T, num_pages = 11 * repeat, 9 * repeat
    S = (n_heads + 2 * n_kv) * hd + 8
    qkv = rnd((T, S), dtype, 8)
    before = qkv.clone()
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 5, 6, 7, 300, 301] * repeat, dtype=torch.int32, device=DEV)
    positions = positions + 13 * torch.arange(T, dtype=torch.int32, device=DEV) // 11
    slots = torch.randperm(num_pages * page_size, generator=torch.Generator().manual_seed(9))[:T]
    if repeat > 1 and page_size == 16:
        # groups of 16 tokens that fill a page in order (their values are written by the kernel that
        # transposes whole pages), and one that does so but for two tokens in each other's places
        taken = [3, 1, 5]
        rest = [int(x) for x in slots if int(x) // 16 not in taken]
        run = lambda pg: [pg * 16 + j for j in range(16)]
        swapped = run(5); swapped[4], swapped[9] = swapped[9], swapped[4]
        slots = torch.tensor((run(3) + run(1) + swapped + rest)[:T])
    slots = slots.to(torch.int32).to(DEV)
    inv_freq = plain_inv_freq(rot, theta, scaling).to(DEV)
    kc = torch.zeros((num_pages, n_kv, page_size, hd), dtype=dtype, device=DEV)
    vc = torch.zeros((num_pages, n_kv, hd, page_size), dtype=dtype, device=DEV)
    kernels().rope_kv_write(qkv, positions, slots, inv_freq, rot, layout == "interleaved", kc, vc,
                            n_heads, n_kv, hd, page_size, num_pages, True)
    b = before.double().cpu()
    q = b[:, :n_heads * hd].view(T, n_heads, hd)
    k = b[:, n_heads * hd:(n_heads + n_kv) * hd].view(T, n_kv, hd)
    v = b[:, (n_heads + n_kv) * hd:(n_heads + 2 * n_kv) * hd].view(T, n_kv, hd)
    qr = plain_rope(q, positions.cpu(), inv_freq.cpu(), layout)
    kr = plain_rope(k, positions.cpu(), inv_freq.cpu(), layout)
    floor = 1e-6 if dtype == torch.float32 else 1e-3
    got_q = qkv[:, :n_heads * hd].double().cpu().view(T, n_heads, hd)
    assert ((got_q - qr).abs() <= out_tol(qr, dtype, floor)).all()
    assert torch.equal(qkv[:, (n_heads + 2 * n_kv) * hd:], before[:, (n_heads + 2 * n_kv) * hd:]), "padding touched"
    page, off = (slots // page_size).long().cpu(), (slots % page_size).long().cpu()
    got_k = kc.double().cpu()[page, :, off, :]
    got_v = vc.double().cpu()[page, :, :, off]
    assert ((got_k - kr).abs() <= out_tol(kr, dtype, floor)).all()
    assert torch.equal(got_v, v), "values are copied unchanged"
    written = torch.zeros(num_pages * page_size, dtype=torch.bool)
    written[slots.long().cpu()] = True
    kflat = kc.cpu().permute(0, 2, 1, 3).reshape(num_pages * page_size, -1)
    vflat = vc.cpu().permute(0, 3, 1, 2).reshape(num_pages * page_size, -1)
    assert (kflat[~written] == 0).all() and (vflat[~written] == 0).all(), "a slot that no token maps to was written"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,rot,layout,page_size", [
    (4, 2, 16, 16, "split_half", 4), (3, 1, 32, 32, "split_half", 16), (5, 5, 48, 48, "interleaved", 16),
    (6, 2, 80, 32, "split_half", 8), (2, 1, 128, 128, "interleaved", 16), (8, 2, 64, 0, "split_half", 16)])
def test_rope_kv_write(dtype, n_heads, n_kv, hd, rot, layout, page_size):
    _rope_case(dtype, n_heads, n_kv, hd, rot, layout, page_size)


@pytest.mark.parametrize("n_heads,n_kv,hd,rot,page_size", [(5, 5, 48, 48, 16), (2, 1, 128, 128, 16), (8, 2, 64, 32, 16),
                                                           (32, 8, 128, 128, 16), (3, 1, 80, 0, 8),
                                                           (20, 20, 32, 32, 16)])    # more kv heads than a page has tokens' blocks to share them out to
def test_rope_kv_write_many_tokens(n_heads, n_kv, hd, rot, page_size):
    _rope_case(torch.bfloat16, n_heads, n_kv, hd, rot, "interleaved", page_size, repeat=4)
    _rope_case(torch.float32, n_heads, n_kv, hd, rot, "interleaved", page_size, repeat=4)


def test_rope_kv_write_llama3_scaling():
    _rope_case(torch.float32, 4, 2, 64, 64, "split_half", 16, theta=500000.0,
               scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                            original_max_position_embeddings=64))


class PagedCase:
    """Sequences with keys and values scattered over shuffled pages."""

    def __init__(self, dtype, lens, n_heads, n_kv, hd, page_size, seed=0, extra_pages=3):
        self.dtype, self.lens, self.n_heads, self.n_kv, self.hd, self.ps = dtype, lens, n_heads, n_kv, hd, page_size
        g = torch.Generator().manual_seed(seed)
        pages_per = [-(-n // page_size) for n in lens]
        self.num_pages = sum(pages_per) + extra_pages
        self.k = [torch.randn((n, n_kv, hd), generator=g).to(dtype) for n in lens]
        self.v = [torch.randn((n, n_kv, hd), generator=g).to(dtype) for n in lens]
        perm = torch.randperm(self.num_pages, generator=g).tolist()
        self.width = max(pages_per)
        self.tables = torch.zeros((len(lens), self.width), dtype=torch.int32)
        self.kc = torch.zeros((self.num_pages, n_kv, page_size, hd), dtype=dtype)
        self.vc = torch.zeros((self.num_pages, n_kv, hd, page_size), dtype=dtype)
        at = 0
        for r, n in enumerate(lens):
            for i in range(pages_per[r]):
                page = perm[at]; at += 1
                self.tables[r, i] = page
                lo, hi = i * page_size, min((i + 1) * page_size, n)
                self.kc[page, :, :hi - lo, :] = self.k[r][lo:hi].permute(1, 0, 2)
                self.vc[page, :, :, :hi - lo] = self.v[r][lo:hi].permute(1, 2, 0)

    def run(self, q_list, q_pos_list, window=0, scale=None, scratch_floats=1 << 22, bound=None, n_single=-1, single_keys=0):
        """q_list[r]: [n_r, heads, hd] queries of request r at positions q_pos_list[r]."""
        scale = 1.0 / math.sqrt(self.hd) if scale is None else scale
        q = torch.cat(q_list).reshape(-1, self.n_heads * self.hd).to(DEV)
        T = q.shape[0]
        entry = torch.cat([torch.full((len(p),), r, dtype=torch.int32) for r, p in enumerate(q_pos_list)]).to(DEV)
        pos = torch.cat([torch.tensor(p, dtype=torch.int32) for p in q_pos_list]).to(DEV)
        lens_now = [max(p) + 1 if len(p) else 1 for p in q_pos_list]      # (an entry without tokens: any length will do)
        counts = [len(p) for p in q_pos_list]
        q_starts = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device=DEV)
        seq_lens = torch.tensor(lens_now, dtype=torch.int32, device=DEV)
        out = torch.zeros((T, self.n_heads * self.hd), dtype=self.dtype, device=DEV)
        scratch = torch.empty(scratch_floats, dtype=torch.float32, device=DEV)
        kernels().attention(q, out, self.kc.to(DEV), self.vc.to(DEV), self.tables.to(DEV), entry, pos, q_starts, seq_lens,
                            self.n_heads, self.n_kv, self.hd, self.ps, self.num_pages, window, scale, scratch,
                            max(lens_now) if bound is None else bound, n_single, single_keys)
        return out.cpu().view(T, self.n_heads, self.hd)

    def reference(self, r, q, positions, window=0, scale=None):
        """Plain attention of request r's queries, each over keys 0..its position."""
        outs = []
        for i, p in enumerate(positions):
            n = p + 1
            if n > 6000:        # the one row of the same formula: the table of all rows' scores would take gigabytes
                G = self.n_heads // self.n_kv
                sc = 1.0 / math.sqrt(self.hd) if scale is None else scale
                s = torch.einsum("hd,nhd->hn", q[i].double(), self.k[r][:n].double().repeat_interleave(G, dim=1)) * sc
                if window and n > window:
                    s[:, :n - window] = -math.inf
                w = torch.softmax(s, dim=-1)
                outs.append(torch.einsum("hn,nhd->hd", w, self.v[r][:n].double().repeat_interleave(G, dim=1)))
                continue
            qq = torch.zeros((n, self.n_heads, self.hd), dtype=torch.float64)
            qq[-1] = q[i].double()
            o = plain_attention(qq, self.k[r][:n].double(), self.v[r][:n].double(), scale, window)
            outs.append(o[-1])
        return torch.stack(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,ps", [(8, 2, 128, 16), (6, 3, 48, 8)])
def test_attention_as_many_tokens_as_entries_but_not_one_each(dtype, n_heads, n_kv, hd, ps):
    """Entries of two tokens and of none come to as many tokens as entries, as single tokens would: the kernels
    treat a batch as single tokens only on the caller's word (n_single == n_entries), never by that count, and a
    caller that claims it for such a batch is refused."""
    lens = [40, 25, 9, 33]
    case = PagedCase(dtype, lens, n_heads, n_kv, hd, ps, seed=3)
    g = torch.Generator().manual_seed(2)
    q_pos = [[38, 39], [], [7, 8], []]
    qs = [torch.randn((len(p), n_heads, hd), generator=g).to(dtype) for p in q_pos]
    floor = 2e-6 if dtype == torch.float32 else 4e-3
    for n_single in (-1, 0):
        got = case.run(qs, q_pos, n_single=n_single)
        at = 0
        for r, p in enumerate(q_pos):
            if p:
                ref = case.reference(r, qs[r], p)
                err = (got[at:at + len(p)].double() - ref).abs()
                assert (err <= out_tol(ref, dtype, floor)).all(), f"n_single {n_single}, entry {r}: max err {float(err.max())}"
                at += len(p)
    q_pos = [[38, 39], [5], [7, 8], [3]]                                  # four entries, six tokens
    qs = [torch.randn((len(p), n_heads, hd), generator=g).to(dtype) for p in q_pos]
    with pytest.raises(KernelError, match="every entry is said to bring one token"):
        case.run(qs, q_pos, n_single=4)


ATTN_SHAPES = [(4, 2, 16, 4), (3, 1, 32, 16), (8, 8, 64, 16), (8, 2, 128, 16), (6, 3, 48, 8), (5, 1, 80, 16),
               (32, 8, 128, 16), (2, 2, 256, 16),
               # 32-bit tiles on the matrix cores: pages of 4 and 8, head sizes in steps of 32, 3 and 32 heads to a kv head
               (6, 2, 32, 4), (4, 4, 96, 8), (32, 1, 64, 16), (2, 1, 160, 16), (3, 3, 192, 32), (2, 2, 224, 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,hd,ps", ATTN_SHAPES)
def test_attention_mixed_batch(dtype, n_heads, n_kv, hd, ps):
    """A prompt portion, a whole prompt, and two decoding requests in one call."""
    lens = [70, 37, 131, 16]
    case = PagedCase(dtype, lens, n_heads, n_kv, hd, ps, seed=hd)
    g = torch.Generator().manual_seed(1)
    q_pos = [list(range(50, 70)), list(range(0, 37)), [130], [15]]
    qs = [torch.randn((len(p), n_heads, hd), generator=g).to(dtype) for p in q_pos]
    got = case.run(qs, q_pos)
    at = 0
    floor = 2e-6 if dtype == torch.float32 else 4e-3
    for r, p in enumerate(q_pos):
        ref = case.reference(r, qs[r], p)
        err = (got[at:at + len(p)].double() - ref).abs()
        assert (err <= out_tol(ref, dtype, floor)).all(), f"request {r}: max err {float(err.max())}"
        at += len(p)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd,ps,n", [(64, 16, 700), (128, 16, 1500), (32, 4, 300),
                                     (128, 16, 2300), (64, 16, 5000),    # more than 16 ranges of 128 keys to merge: the merge kernel's later groups
                                     (128, 16, 8300), (64, 16, 17000), (96, 16, 9000)])   # more than 64 ranges: the merge whose threads share them out
def test_attention_finds_a_far_key(dtype, hd, ps, n):
    """Random keys hide a key that is skipped or read from the wrong page: here one
    early key matches the query so strongly that the output must be its value."""
    n_heads, n_kv = 4, 2
    case = PagedCase(dtype, [n], n_heads, n_kv, hd, ps, seed=3)
    fars = (0, ps - 1, ps, 63, 64, n // 2 + 1, n - 2) + ((2053, n - 300) if n > 2100 else ())    # (one request alone: ranges of 64 keys)
    if n > 8192:        # one key in each of the last ranges of 128, and in ranges that different groups of the merge's threads take
        fars = fars + tuple(n - 1 - 128 * i - 7 * i for i in range(1, 20)) + (129, 1024 + 5, 4096 - 1, 4096, 8191)
    for far in fars:
        q = torch.zeros((1, n_heads, hd))
        q[0, :, :] = case.k[0][far, :, :].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0
        got = case.run([q.to(dtype)], [[n - 1]])
        want = case.v[0][far].float().repeat_interleave(n_heads // n_kv, dim=0)
        ref = case.reference(0, q.to(dtype), [n - 1])
        assert (ref[0].float() - want).abs().max() < 0.05, "the case itself: softmax must be peaked on the far key"
        tol = 1e-4 if dtype == torch.float32 else 2e-2
        assert (got[0].float() - ref[0].float()).abs().max() <= tol, f"far key {far}"


def test_attention_at_131008_keys():
    """One request decoding over 131,008 keys at head size 128 in bfloat16 (134 MB of cache, 8,188 pages scattered
    over the pool, a block table that wide, the most chunks the merge takes): a key that matches the query strongly is
    found wherever it lies (the first and last keys, the edges of pages, of every chunk length and of 65,536), and random
    queries agree with the plain formula."""
    n, n_heads, n_kv, hd, ps = 131008, 8, 2, 128, 16
    case = PagedCase(torch.bfloat16, [n], n_heads, n_kv, hd, ps, seed=23)
    assert case.width == 8188
    fars = (0, 15, 16, 511, 512, 1023, 1024, 32767, 65535, 65536, 65537, 100003, n - 1025, n - 1024, n - 513, n - 17, n - 2, n - 1)
    for far in fars:
        q = (case.k[0][far].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0).unsqueeze(0).to(torch.bfloat16)
        got = case.run([q], [[n - 1]], n_single=1, single_keys=n)
        want = case.v[0][far].float().repeat_interleave(n_heads // n_kv, dim=0)
        ref = case.reference(0, q, [n - 1])[0].float()
        assert (ref - want).abs().max() < 0.05, "the case itself: softmax must be peaked on the far key"
        assert (got[0].float() - ref).abs().max() <= 2e-2, f"far key {far}"
    g = torch.Generator().manual_seed(9)
    for i in range(3):
        # queries of growing length: from nearly uniform weights over all keys to a handful of keys that count
        q = (torch.randn((1, n_heads, hd), generator=g) * (0.5, 1.5, 3.0)[i]).to(torch.bfloat16)
        got = case.run([q], [[n - 1]], n_single=1, single_keys=n)
        ref = case.reference(0, q, [n - 1])[0].float()
        assert (got[0].float() - ref).abs().max() <= 4e-3 + 2e-2 * float(ref.abs().max()), f"random query {i}"


@pytest.mark.parametrize("n_heads,n_kv,hd,window", [(8, 2, 128, 0), (6, 2, 128, 20000), (16, 2, 128, 0)])
def test_attention_prompt_portions_over_long_caches(n_heads, n_kv, hd, window):
    """Prompt portions against caches of 33,000 and 40,000 keys in bfloat16: from 32,768 keys on the tiles' blocks
    have eight waves at head size 128 (with 4, 3 and 8 heads to a kv head here: 64, 80 and 32 tokens a block), and a column's sums
    must be the four-wave blocks' bit for bit.  Portions that end inside a block and one that is a single block's
    worth; every query of the first request matches one key strongly (the first and last it may see, the edges of
    pages and of the 32-key tiles, its own position), so its output must be that key's value; random queries agree
    with the plain formula; and the same portions under a bound below 32,768 keys (the four-wave blocks) give the
    same bits."""
    lens = [33000, 40000, 50]
    case = PagedCase(torch.bfloat16, lens, n_heads, n_kv, hd, 16, seed=41)
    G = n_heads // n_kv
    g = torch.Generator().manual_seed(6)
    counts = [150, 64, 7]
    q_pos = [list(range(n - c, n)) for n, c in zip(lens, counts)]
    qs = [torch.randn((c, n_heads, hd), generator=g).to(torch.bfloat16) for c in counts]
    fars = []
    for i, p in enumerate(q_pos[0]):
        lo = max(0, p + 1 - window) if window else 0
        far = (lo, lo + 1, p, p - 1, 31, 32, 16383, 16384, 32767, 32768, (lo + p) // 2, lo + 15, lo + 16)[i % 13]
        far = min(max(far, lo), p)
        fars.append(far)
        qs[0][i] = (case.k[0][far].float().repeat_interleave(G, dim=0) * 8.0).to(torch.bfloat16)
    got = case.run(qs, q_pos, window=window, n_single=0)
    at = 0
    for r, p in enumerate(q_pos):
        rows = got[at:at + len(p)].float()
        at += len(p)
        pick = range(0, len(p), 2) if r == 0 else (0, len(p) // 2, len(p) - 1)      # (every kind of far key: 2 and 13 share no factor)
        for i in pick:
            ref = case.reference(r, qs[r][i:i + 1], [p[i]], window=window)[0].float()
            if r == 0:
                want = case.v[0][fars[i]].float().repeat_interleave(G, dim=0)
                assert (ref - want).abs().max() < 0.05, "the case itself: softmax must be peaked on the far key"
            assert (rows[i] - ref).abs().max() <= 4e-3 + 2e-2 * float(ref.abs().max()), (r, i)
    # a request of 40,000 keys under a bound of 32,000 would be a caller's mistake, so the four-wave blocks are
    # asked for through the two requests that such a bound fits: the first, cut to 32,000 keys, and the third
    short = [list(range(32000 - 150, 32000)), [], q_pos[2]]
    qs_short = [qs[0], qs[1][:0], qs[2]]
    four = case.run(qs_short, short, window=window, n_single=0, bound=32000)
    eight = case.run(qs_short, short, window=window, n_single=0, bound=32768)
    assert torch.equal(four, eight), "a column's sums do not depend on how many waves share its keys"


@pytest.mark.parametrize("n_heads,n_kv,hd,ps,window", [(8, 2, 128, 16, 0), (3, 3, 64, 8, 0), (6, 2, 96, 16, 300), (32, 1, 32, 4, 0),
                                                        (4, 4, 160, 16, 130), (16, 2, 256, 32, 0)])
def test_attention_float32_decoding_requests(n_heads, n_kv, hd, ps, window):
    """Single tokens in 32-bit: a wave of the matrix-core split takes a chunk of 128 keys for all heads of a kv head (1,
    3, 4, 8 and 32 of them here).  Lengths at and around the chunks' edges, with and without a window whose edge cuts
    a chunk; each query matches one key strongly, at the first and last key it may see and at the chunks' edges, so
    the output must be that key's value; and random queries agree with the plain formula to 32-bit rounding."""
    lens = [1, 127, 128, 129, 256, 257, 700, 1500]
    case = PagedCase(torch.float32, lens, n_heads, n_kv, hd, ps, seed=31)
    G = n_heads // n_kv
    g = torch.Generator().manual_seed(4)
    for shift in range(3):
        qs, fars = [], []
        for r, n in enumerate(lens):
            lo = max(0, n - window) if window else 0
            seen = sorted({e for e in (lo, lo + 1, n - 1, 127, 128, 255, 256, n - 2, (lo + n) // 2) if lo <= e < n})
            far = seen[(r + shift * 2) % len(seen)]
            fars.append(far)
            qs.append((case.k[r][far].repeat_interleave(G, dim=0) * 8.0).unsqueeze(0))
        got = case.run(qs, [[n - 1] for n in lens], window=window, n_single=len(lens), single_keys=sum(lens))
        for r in range(len(lens)):
            want = case.v[r][fars[r]].repeat_interleave(G, dim=0)
            ref = case.reference(r, qs[r], [lens[r] - 1], window=window)[0].float()
            if lens[r] > 1:
                assert (ref - want).abs().max() < 0.05, "the case itself"
            assert (got[r] - ref).abs().max() <= 1e-4, f"request of length {lens[r]}, key {fars[r]}"
    qs = [torch.randn((1, n_heads, hd), generator=g) for _ in lens]
    got = case.run(qs, [[n - 1] for n in lens], window=window, n_single=len(lens), single_keys=sum(lens))
    for r in range(len(lens)):
        ref = case.reference(r, qs[r], [lens[r] - 1], window=window)[0]
        err = (got[r].double() - ref).abs()
        assert (err <= out_tol(ref, torch.float32, 2e-6)).all(), f"request of length {lens[r]}: {float(err.max())}"


@pytest.mark.parametrize("M,N,K", [(3, 48, 64), (8, 4096, 4096), (16, 6144, 2048), (5, 130, 96), (9, 28672, 256), (12, 16400, 128),
                                   (16, 2048, 8192), (7, 5000, 1024), (4, 100, 32)])
def test_gemm_float32_few_rows_on_the_matrix_cores(M, N, K):
    """3 to 16 rows in 32-bit: the product on v_mfma_f32_16x16x4_f32 against float64, every epilogue, rows with a
    stride, weights whose last feature tile is cut by N, and against the walk that takes the same product when the
    matrix cores are switched off (both true 32-bit: they differ by the order of their sums only)."""
    a_full = rnd((M, K + 24), torch.float32, 3)
    a = a_full[:, :K]
    w = rnd((N, K), torch.float32, 4, 0.1)
    acc = a.double().cpu() @ w.double().cpu().T
    k = kernels()
    for epi in (EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU):
        outs = []
        for mfma in (True, False):
            k.allow_mfma = mfma
            try:
                if epi == EPI_ACCUM_F32:
                    out = rnd((M, N), torch.float32, 5)
                    ref = out.double().cpu() + acc
                elif epi == EPI_SWIGLU:
                    out = torch.zeros((M, N // 2), dtype=torch.float32, device=DEV)
                    ref = plain_silu(acc[:, 0::2]) * acc[:, 1::2]
                else:
                    out = torch.zeros((M, N), dtype=torch.float32, device=DEV)
                    ref = acc
                k.gemm(a, w, out, epi)
            finally:
                k.allow_mfma = True
            err = (out.double().cpu() - ref).abs()
            floor = 2e-6 * math.sqrt(K)
            if epi == EPI_SWIGLU:
                floor *= 1 + 0.1 * math.sqrt(K)      # a sum's rounding error is multiplied by the other factor, of size 0.1 sqrt(K)
            assert (err <= out_tol(ref, torch.float32, floor)).all(), (epi, mfma, float(err.max()))
            outs.append(out.cpu())
        assert ((outs[0] - outs[1]).abs().double() <= 2 * out_tol(ref, torch.float32, floor)).all()


def test_attention_chunk_rule_and_its_scratch():
    """The keys per wave that the split takes: a power of two from 64 to 1024 whatever the host says about the
    keys; never under what the scratch is sized by (the answer for one key); and the same results whichever chunk
    the number of keys leads to, with a scratch of exactly the size the library asks for."""
    k = kernels()
    for n, kv, hd, bound in ((1, 8, 128, 2048), (8, 8, 64, 2048), (12, 2, 96, 4096), (64, 8, 128, 2048), (200, 4, 256, 8192), (1, 1, 32, 131072),
                             (3, 8, 80, 40000), (33, 8, 64, 2048)):
        least = k.attention_split_chunk(n, kv, hd, bound, 1)
        for keys in (0, 1, n * bound // 16, n * bound // 3, n * bound, 10 * n * bound):
            c = k.attention_split_chunk(n, kv, hd, bound, keys)
            assert c in (64, 128, 256, 512, 1024) and c >= least, (n, kv, bound, keys, c, least)
            assert -(-bound // c) <= 256 or c == 1024
    n_heads, n_kv, hd, ps = 8, 8, 128, 16
    lens = [1500, 700, 1290, 40, 2047, 900, 1100, 333, 1999, 1203]
    case = PagedCase(torch.bfloat16, lens, n_heads, n_kv, hd, ps, seed=41)
    g = torch.Generator().manual_seed(3)
    qs = [torch.randn((1, n_heads, hd), generator=g).to(torch.bfloat16) for _ in lens]
    pos = [[n - 1] for n in lens]
    refs = [case.reference(r, qs[r], pos[r])[0].float() for r in range(len(lens))]
    seen = set()
    for keys in (0, 1, sum(lens), 40 * sum(lens), 400 * sum(lens)):
        c = k.attention_split_chunk(len(lens), n_kv, hd, 2048, keys)
        seen.add(c)
        need = k.attention_scratch_floats(len(lens), n_heads, hd, 2048, n_kv, len(lens))
        assert need >= len(lens) * n_heads * -(-2048 // c) * (hd + 2)
        got = case.run(qs, pos, scratch_floats=need, bound=2048, n_single=len(lens), single_keys=keys)
        for r in range(len(lens)):
            assert (got[r].float() - refs[r]).abs().max() <= 2e-2, f"{keys} keys, request {r}"
    assert len(seen) >= 2, "the case itself: more than one chunk"


@pytest.mark.parametrize("portion", [False, True])
def test_attention_long_caches_with_a_window(portion):
    """Two decoding requests over long caches with a window of 8500 keys (more than 64 ranges to merge, the first of
    them cut by the window's edge), with and without a prompt portion beside them: a key just inside the window is
    found, one just outside it is not seen."""
    n_heads, n_kv, hd, ps, window = 8, 2, 128, 16, 8500
    lens = [12000, 9100] + ([40] if portion else [])
    case = PagedCase(torch.bfloat16, lens, n_heads, n_kv, hd, ps, seed=29)
    g = torch.Generator().manual_seed(5)
    for inside in (True, False):
        qs, pos, fars = [], [], []
        for r, n in enumerate(lens[:2]):
            far = n - window + (0 if inside else -1)
            fars.append(far)
            qs.append((case.k[r][far].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0).unsqueeze(0).to(torch.bfloat16))
            pos.append([n - 1])
        if portion:
            qs.append(torch.randn((40, n_heads, hd), generator=g).to(torch.bfloat16))
            pos.append(list(range(40)))
        got = case.run(qs, pos, window=window)
        for r in range(2):
            want = case.v[r][fars[r]].float().repeat_interleave(n_heads // n_kv, dim=0)
            ref = case.reference(r, qs[r], pos[r], window=window)[0].float()
            assert ((ref - want).abs().max() < 0.05) == inside, "the case itself"
            assert (got[r].float() - ref).abs().max() <= 2e-2, f"request of length {lens[r]}, key {fars[r]}"


@pytest.mark.parametrize("window", [0, 300])
@pytest.mark.parametrize("portion", [False, True])
def test_attention_few_decoding_requests(window, portion):
    """With few decoding requests a wave of the split takes 64 keys.  Each request's query matches one key
    strongly, at the edges of such ranges and of the window: the output must be that key's value, with and
    without a prompt portion in the same call (with one, a wave looks its token up instead of taking the
    entry's number), and agree with the plain implementation."""
    n_heads, n_kv, hd, ps = 8, 2, 128, 16
    g = torch.Generator().manual_seed(7 + window)
    lens = [130, 1000, 2047, 64, 65] + ([90] if portion else [])
    case = PagedCase(torch.bfloat16, lens, n_heads, n_kv, hd, ps, seed=13)
    edges = [0, 63, 64, 65, 127, 128, 191, 192, 959, 960, 1983, 1984]
    n_dec = 5
    for shift in range(4):
        qs, pos, fars = [], [], []
        for r, n in enumerate(lens[:n_dec]):
            lo = max(0, n - window) if window else 0
            seen = [e for e in edges + [lo, lo + 1, n - 1] if lo <= e < n]
            far = seen[(5 * r + 3 * shift) % len(seen)]
            fars.append(far)
            qs.append((case.k[r][far].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0).unsqueeze(0).to(torch.bfloat16))
            pos.append([n - 1])
        if portion:
            qs.append(torch.randn((30, n_heads, hd), generator=g).to(torch.bfloat16))
            pos.append(list(range(60, 90)))
        got = case.run(qs, pos, window=window)
        for r in range(n_dec):
            want = case.v[r][fars[r]].float().repeat_interleave(n_heads // n_kv, dim=0)
            ref = case.reference(r, qs[r], pos[r], window=window)[0].float()
            assert (ref - want).abs().max() < 0.05, "the case itself"
            assert (got[r].float() - ref).abs().max() <= 2e-2, f"request of length {lens[r]}, key {fars[r]}"
        if portion:
            ref = case.reference(n_dec, qs[-1], pos[-1], window=window).float()
            assert (got[n_dec:].float() - ref).abs().max() <= 3e-2


@pytest.mark.parametrize("n_req,hd", [(3, 128), (20, 128), (70, 64), (70, 128), (160, 128)])
def test_attention_decoding_requests_a_few_keys_past_a_chunk(n_req, hd):
    """Lengths a few keys (and a few more than a few) past multiples of every chunk length: a request's last chunk
    then holds a handful of keys.  The strong key among those last keys, at the first of them and just before: the
    output must be that key's value, for every number of requests (which decides the chunk length)."""
    n_heads, n_kv, ps = 8, 2, 16
    tails = [1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129]
    lens = [(64 << (r % 5)) * (1 + r % 2) + tails[r % len(tails)] for r in range(n_req)]
    case = PagedCase(torch.bfloat16, lens, n_heads, n_kv, hd, ps, seed=17)
    for which in range(3):
        qs, fars = [], []
        for r, n in enumerate(lens):
            t = tails[r % len(tails)]
            far = (n - 1, n - t, n - t - 1)[which]
            fars.append(far)
            qs.append((case.k[r][far].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0).unsqueeze(0).to(torch.bfloat16))
        got = case.run(qs, [[n - 1] for n in lens], n_single=n_req, single_keys=sum(lens))
        for r in range(n_req):
            want = case.v[r][fars[r]].float().repeat_interleave(n_heads // n_kv, dim=0)
            assert (got[r].float() - want).abs().max() < 0.07, f"request {r} of length {lens[r]}, key {fars[r]}"
            if r < 6:
                ref = case.reference(r, qs[r], [lens[r] - 1])[0].float()
                assert (got[r].float() - ref).abs().max() <= 2e-2, f"request {r}"


@pytest.mark.parametrize("n_heads,n_kv,hd", [(1, 1, 128), (5, 1, 64), (16, 2, 32), (16, 1, 128), (12, 2, 96), (20, 1, 64), (40, 2, 128),
                                             (9, 3, 192), (4, 2, 256), (32, 8, 128)])
@pytest.mark.parametrize("window", [0, 70])
def test_attention_decoding_every_group_size(n_heads, n_kv, hd, window):
    """Decoding requests with a random query for every head, 1 to 20 heads to a kv head (up to 16 a wave of the split
    takes 16 query columns, beyond that 32), every head size the split has a kernel for, lengths around the edges of
    32-key steps and of chunks, with and without a window: every head against the plain implementation."""
    ps = 16
    lens = [1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 257, 500, 777, 1030]
    case = PagedCase(torch.bfloat16, lens, n_heads, n_kv, hd, ps, seed=hd + n_heads)
    g = torch.Generator().manual_seed(n_heads * 7 + hd)
    qs = [torch.randn((1, n_heads, hd), generator=g).to(torch.bfloat16) for _ in lens]
    pos = [[n - 1] for n in lens]
    got = case.run(qs, pos, window=window, n_single=len(lens), single_keys=sum(min(n, window) if window else n for n in lens))
    for r in range(len(lens)):
        ref = case.reference(r, qs[r], pos[r], window=window)[0].float()
        assert (got[r].float() - ref).abs().max() <= 2e-2, f"request {r} of length {lens[r]}"


@pytest.mark.parametrize("window", [0, 300])
@pytest.mark.parametrize("n_req", [70, 150])
def test_attention_many_decoding_requests(n_req, window):
    """With many decoding requests a wave of the split takes a longer range of keys (256 to 1024
    instead of 128).  Each request's query matches one key strongly, chosen at the edges of such
    ranges (and of the window, if there is one) where the request is long enough: the output
    must be that key's value."""
    n_heads, n_kv, hd, ps = 16, 8, 64, 16
    g = torch.Generator().manual_seed(n_req)
    lens = [int(x) for x in torch.randint(5, 1500, (n_req,), generator=g)]
    lens[0], lens[1] = 1499, 1025
    case = PagedCase(torch.bfloat16, lens, n_heads, n_kv, hd, ps, seed=11)
    edges = [0, 127, 128, 255, 256, 511, 512, 1023, 1024, 1279, 1280]
    qs, fars = [], []
    for r, n in enumerate(lens):
        lo = max(0, n - window) if window else 0
        seen = [e for e in edges + [lo, lo + 1, n - 1] if lo <= e < n]
        far = seen[r % len(seen)] if r % 3 else int(torch.randint(lo, n, (1,), generator=g))
        fars.append(far)
        qs.append((case.k[r][far].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0).unsqueeze(0).to(torch.bfloat16))
    got = case.run(qs, [[n - 1] for n in lens], window=window)
    for r in range(n_req):
        want = case.v[r][fars[r]].float().repeat_interleave(n_heads // n_kv, dim=0)
        if r < 12:          # the case itself, and the kernel against the plain implementation
            ref = case.reference(r, qs[r], [lens[r] - 1], window=window)[0].float()
            assert (ref - want).abs().max() < 0.05
            assert (got[r].float() - ref).abs().max() <= 2e-2, f"request {r}"
        assert (got[r].float() - want).abs().max() < 0.07, f"request {r} of length {lens[r]}, key {fars[r]}"


@pytest.mark.parametrize("dtype,n_heads,n_kv,hd,ps", [(torch.bfloat16, 8, 2, 128, 16), (torch.bfloat16, 8, 2, 96, 16),
                                                     (torch.float32, 4, 2, 64, 16), (torch.bfloat16, 8, 8, 64, 16)])
def test_attention_prompt_portions_among_many_entries(dtype, n_heads, n_kv, hd, ps):
    """A serving step: prompt portions at the start, in the middle and at the end of 150 entries that bring one
    token each.  A tile's entry is looked up 64 entries at a time (the kernels with shared tiles, those without, and the
    32-bit tiles each do it): every portion's rows against the plain implementation, and some of the single tokens."""
    g = torch.Generator().manual_seed(hd)
    n_single = 150
    single_lens = [int(x) for x in torch.randint(3, 200, (n_single,), generator=g)]
    portions = {0: (40, 70), 77: (0, 33), 151: (100, 45), 152: (5, 1)}      # entry -> (start, tokens); the last brings one token of a prompt
    lens, counts = [], []
    singles = iter(single_lens)
    for e in range(n_single + len(portions)):
        if e in portions:
            start, cnt = portions[e]
            lens.append(start + cnt); counts.append(cnt)
        else:
            lens.append(next(singles)); counts.append(1)
    case = PagedCase(dtype, lens, n_heads, n_kv, hd, ps, seed=hd + 1)
    qs = [torch.randn((c, n_heads, hd), generator=g).to(dtype) for c in counts]
    pos = [list(range(n - c, n)) for n, c in zip(lens, counts)]
    got = case.run(qs, pos, n_single=sum(1 for c in counts if c == 1))
    at = [0]
    for c in counts:
        at.append(at[-1] + c)
    floor = 2e-6 if dtype == torch.float32 else 4e-3
    for e in list(portions) + [1, 63, 64, 76, 78, 127, 128, 150]:
        ref = case.reference(e, qs[e], pos[e])
        err = (got[at[e]:at[e + 1]].double() - ref).abs()
        assert (err <= out_tol(ref, dtype, floor)).all(), f"entry {e} ({counts[e]} tokens): max err {float(err.max())}"


@pytest.mark.parametrize("window", [0, 200])
@pytest.mark.parametrize("dtype,n_heads,n_kv,hd,ps", [(torch.float32, 4, 2, 64, 16), (torch.float32, 3, 1, 20, 4),
                                                     (torch.bfloat16, 6, 3, 48, 8), (torch.bfloat16, 5, 5, 80, 16),
                                                     (torch.float32, 2, 2, 18, 4), (torch.float32, 8, 2, 32, 16),
                                                     (torch.bfloat16, 8, 1, 48, 8)])
def test_attention_plain_kernel_splits_decoding_requests(dtype, n_heads, n_kv, hd, ps, window):
    """Head and page sizes (and the 32-bit type) that the matrix-core kernels do not take: decoding
    requests are shared out over waves in chunks of 128 keys and merged; a prompt portion rides in
    the same call.  Each decoding query matches one key strongly, at the edges of chunks and of the
    window: the output must be that key's value, and agree with the plain implementation."""
    g = torch.Generator().manual_seed(hd + window)
    lens = [1, 127, 128, 129, 256, 257, 700, 90]
    case = PagedCase(dtype, lens, n_heads, n_kv, hd, ps, seed=hd)
    edges = [0, 63, 64, 127, 128, 255, 256, 383, 384, 511, 512, 639, 640]
    qs, pos, fars = [], [], []
    for r, n in enumerate(lens[:-1]):
        lo = max(0, n - window) if window else 0
        seen = [e for e in edges + [lo, lo + 1, n - 1] if lo <= e < n]
        far = seen[(3 * r + 1) % len(seen)]
        fars.append(far)
        qs.append((case.k[r][far].float().repeat_interleave(n_heads // n_kv, dim=0) * 6.0).unsqueeze(0).to(dtype))
        pos.append([n - 1])
    qs.append(torch.randn((30, n_heads, hd), generator=g).to(dtype))       # a prompt portion of the last request
    pos.append(list(range(60, 90)))
    got = case.run(qs, pos, window=window)
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    for r in range(len(lens) - 1):
        ref = case.reference(r, qs[r], pos[r], window=window)[0].float()
        assert (got[r].float() - ref).abs().max() <= tol, f"request of length {lens[r]}, key {fars[r]}"
        if lens[r] > 1 and hd >= 48:        # (short heads cannot make one key stand out among hundreds)
            want = case.v[r][fars[r]].float().repeat_interleave(n_heads // n_kv, dim=0)
            assert (ref - want).abs().max() < 0.1, "the case itself"
    ref = case.reference(len(lens) - 1, qs[-1], pos[-1], window=window).float()
    assert (got[len(lens) - 1:].float() - ref).abs().max() <= tol


@pytest.mark.parametrize("dtype,n_heads,n_kv,hd,ps", [(torch.float32, 8, 2, 32, 16), (torch.float32, 4, 2, 64, 16),
                                                     (torch.bfloat16, 16, 2, 48, 8)])
def test_attention_plain_kernel_many_decoding_requests(dtype, n_heads, n_kv, hd, ps):
    """With enough decoding requests the plain kernel's waves each serve all heads of a kv head
    (4, 2 and 8 here): every request against the plain implementation, a window on."""
    n_req, window = 56, 300
    g = torch.Generator().manual_seed(hd)
    lens = [int(x) for x in torch.randint(1, 700, (n_req,), generator=g)]
    lens[0], lens[1], lens[2] = 699, 128, 129
    case = PagedCase(dtype, lens, n_heads, n_kv, hd, ps, seed=3)
    qs = [torch.randn((1, n_heads, hd), generator=g).to(dtype) for _ in lens]
    got = case.run(qs, [[n - 1] for n in lens], window=window)
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    for r in range(n_req):
        ref = case.reference(r, qs[r], [lens[r] - 1], window=window)[0].float()
        assert (got[r].float() - ref).abs().max() <= tol, f"request {r} of length {lens[r]}"


@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("dtype,n_heads,n_kv,hd,ps", [(torch.float32, 8, 2, 32, 16), (torch.float32, 4, 2, 64, 4),
                                                     (torch.bfloat16, 16, 2, 48, 8)])
def test_attention_plain_kernel_long_prompt_portion(dtype, n_heads, n_kv, hd, ps, window):
    """A prompt portion long enough that the plain kernel's waves each serve all heads of a kv head
    (4, 2 and 8 here), a whole short prompt and a decoding request beside it."""
    g = torch.Generator().manual_seed(hd + window)
    lens = [400, 9, 200]
    case = PagedCase(dtype, lens, n_heads, n_kv, hd, ps, seed=5)
    pos = [list(range(80, 400)), list(range(0, 9)), [199]]
    qs = [torch.randn((len(p), n_heads, hd), generator=g).to(dtype) for p in pos]
    got = case.run(qs, pos, window=window)
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    at = 0
    for r, p in enumerate(pos):
        ref = case.reference(r, qs[r], p, window=window).float()
        assert (got[at:at + len(p)].float() - ref).abs().max() <= tol, f"request {r}"
        at += len(p)


@pytest.mark.parametrize("dtype,ps", [(torch.bfloat16, 16), (torch.float32, 16), (torch.float32, 4), (torch.float32, 32)])
@pytest.mark.parametrize("hd", [64, 96, 128, 256])
def test_attention_prompt_portion_finds_far_keys(hd, dtype, ps):
    """A portion of a prompt far into a long sequence (page numbers are fetched 64 at a time, tiles
    are loaded several ahead): each of its tokens matches one key, early, late or at a page's or a
    fetch's edge, so strongly that its output must be that key's value.  In 32-bit the tiles of the
    matrix cores' 32-bit kernel, with pages of other sizes too."""
    n_heads, n_kv, n = 4, 2, 2300
    case = PagedCase(dtype, [n], n_heads, n_kv, hd, ps, seed=6)
    far = [0, 15, 16, 31, 32, 500, 1023, 1024, 1025, 1039, 1040, 1100, 2047, 2048, 2063, 2064, 2200, 2251, 2252, 2260]
    positions = list(range(n - 40, n))
    q = torch.randn((len(positions), n_heads, hd), generator=torch.Generator().manual_seed(7)) * 0.1
    for i, f in enumerate(far):
        q[2 * i] = case.k[0][f, :, :].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0
    got = case.run([q.to(dtype)], [positions])
    ref = case.reference(0, q.to(dtype), positions)
    for i, f in enumerate(far):
        want = case.v[0][f].float().repeat_interleave(n_heads // n_kv, dim=0)
        assert (ref[2 * i].float() - want).abs().max() < 0.05, "the case itself: softmax must be peaked on the far key"
    assert (got.float() - ref.float()).abs().max() <= (2e-2 if dtype == torch.bfloat16 else 2e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("hd", [64, 128, 256, 96])
@pytest.mark.parametrize("window", [1, 31, 32, 33, 100, 1200])
def test_attention_prompt_portion_with_a_window(hd, window, dtype):
    """Portions of a prompt under a sliding window, with the tiled kernels: random queries against
    the plain function, and for each token the key just outside its window must not be seen."""
    n_heads, n_kv, ps, n = 4, 2, 16, 1500
    case = PagedCase(dtype, [n], n_heads, n_kv, hd, ps, seed=8)
    positions = list(range(n - 70, n))
    q = torch.randn((len(positions), n_heads, hd), generator=torch.Generator().manual_seed(9))
    for i in range(0, len(positions), 7):            # these tokens look hard at the key just outside their window
        outside = positions[i] - window
        if outside >= 0:
            q[i] = case.k[0][outside, :, :].float().repeat_interleave(n_heads // n_kv, dim=0) * 8.0
    got = case.run([q.to(dtype)], [positions], window=window)
    ref = case.reference(0, q.to(dtype), positions, window=window)
    assert (got.float() - ref.float()).abs().max() <= (2.5e-2 if dtype == torch.bfloat16 else 2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 16, 17, 64])
def test_attention_window_edge(dtype, window):
    """The key just outside the window must not be seen, the one just inside must."""
    n_heads, n_kv, hd, ps, n = 2, 1, 32, 16, 90
    case = PagedCase(dtype, [n], n_heads, n_kv, hd, ps, seed=4)
    p = n - 1
    for key, visible in ((p - window, False), (p - window + 1, True)):
        if key < 0:
            continue
        q = torch.zeros((1, n_heads, hd))
        q[0] = case.k[0][key, 0].float() * 8.0
        got = case.run([q.to(dtype)], [[p]], window=window)
        ref = case.reference(0, q.to(dtype), [p], window=window)
        tol = 1e-4 if dtype == torch.float32 else 2e-2
        assert (got[0].float() - ref[0].float()).abs().max() <= tol
        near = (got[0, 0].float() - case.v[0][key, 0].float()).abs().max() < 0.1
        assert bool(near) == visible, f"window {window}: key {key} should {'' if visible else 'not '}be visible"


def test_attention_pages_may_move():
    """The same keys on other pages give the same result (bitwise: same order of sums)."""
    a = PagedCase(torch.float32, [100], 4, 2, 32, 16, seed=5, extra_pages=1)
    b = PagedCase(torch.float32, [100], 4, 2, 32, 16, seed=5, extra_pages=9)
    assert not torch.equal(a.tables, b.tables[:, :a.tables.shape[1]])
    g = torch.Generator().manual_seed(2)
    q = torch.randn((3, 4, 32), generator=g)
    assert torch.equal(a.run([q], [[97, 98, 99]]), b.run([q], [[97, 98, 99]]))


def test_argmax_rows():
    V = 1003
    logits = rnd((6, V + 5), torch.float32, 11)[:, :V]
    logits[1, 77] = 50.0
    logits[2, [5, 900]] = 60.0          # a tie: the lower index wins
    logits[3, V - 1] = 70.0
    logits[4] = -3.0                    # all equal
    out = torch.zeros(6, dtype=torch.int32, device=DEV)
    kernels().argmax_rows(logits, out)
    want = [int(logits[0].argmax()), 77, 5, V - 1, 0, int(logits[5].argmax())]
    assert out.tolist() == want


def test_argmax_rows_long_rows_in_parts():
    V = 128256
    logits = rnd((5, V), torch.float32, 12)
    logits[1, [4007, 4008, 100000]] = 50.0      # a tie across the parts of the row
    logits[2, V - 1] = 60.0
    logits[3] = 1.5
    scratch = torch.zeros(5 * 64, dtype=torch.int32, device=DEV)
    for s in (scratch, None):
        out = torch.zeros(5, dtype=torch.int32, device=DEV)
        kernels().argmax_rows(logits, out, s)
        assert out.tolist() == [int(logits[0].argmax()), 4007, V - 1, 0, int(logits[4].argmax())]


def _words(rows):
    """[(uniform, temperature, top_k, top_p)] -> the int32 words the sampler reads."""
    w = torch.zeros((len(rows), 4), dtype=torch.int32)
    for i, (u, t, k, p) in enumerate(rows):
        f = torch.tensor([u, t, p], dtype=torch.float32).view(torch.int32)
        w[i, 0], w[i, 1], w[i, 2], w[i, 3] = f[0], f[1], k, f[2]
    return w.to(DEV)


@pytest.mark.parametrize("V", [1003, 5000, 140004])    # a row with a tail, rows read 16 bytes a lane, stretches too long for one walk
def test_sample_rows_against_plain(V):
    """The token must be the one whose interval of the plain implementation's cumulative
    distribution (float64) holds the uniform; a uniform within 1e-5 of an interval's edge
    may fall to either side, since the kernel sums in 32-bit."""
    from plain_llama import plain_probabilities
    g = torch.Generator().manual_seed(V)
    settings = [(0.8, 0, 1.0), (0.7, 40, 0.9), (1.3, 5, 1.0), (0.5, 0, 0.8), (1.0, 3000, 0.95), (2.0, 1, 1.0),
                (0.9, 40, 0.3), (1.0, 0, 0.999)]
    rows, logit_rows = [], []
    for (t, k, p) in settings:
        for _ in range(6 if V < 100000 else 2):
            rows.append((float(torch.rand(1, generator=g)), t, k, p))
            logit_rows.append(torch.randn(V, generator=g) * 3.0)
    rows.append((0.3, 0.0, 0, 1.0))                     # a greedy row among the others
    logit_rows.append(torch.randn(V, generator=g))
    logits = torch.stack(logit_rows).to(DEV)
    out = torch.zeros(len(rows), dtype=torch.int32, device=DEV)
    kernels().sample_rows(logits, _words(rows), out)
    out = out.tolist()
    for i, (u, t, k, p) in enumerate(rows):
        if t == 0.0:
            assert out[i] == int(logit_rows[i].argmax())
            continue
        prob = plain_probabilities(logit_rows[i], t, k, p)
        cum = torch.cumsum(prob, 0)
        tok = out[i]
        assert prob[tok] > 0, f"row {i}: token {tok} is outside the kept set (T={t} k={k} p={p})"
        lo = float(cum[tok] - prob[tok])
        assert lo - 1e-5 <= u < float(cum[tok]) + 1e-5, f"row {i}: u={u} not in [{lo}, {float(cum[tok])}) of token {tok}"


def test_sample_rows_ties_and_edges():
    V = 300
    logits = torch.full((4, V), -2.0)
    logits[0, [10, 20, 30]] = 5.0          # three equal maxima, top_k 2: the two lowest indices stay
    logits[1, [10, 20, 30]] = 5.0          # top_p cut through equal values
    logits[2, 7] = 9.0                     # u close to 1 still lands on a kept token
    logits[3, :] = 0.0                     # uniform distribution, top_k 1 -> index 0
    rows = [(0.99, 1.0, 2, 1.0), (0.6, 1.0, 0, 0.5), (0.999999, 1.0, 5, 0.9), (0.5, 1.0, 1, 1.0)]
    out = torch.zeros(4, dtype=torch.int32, device=DEV)
    kernels().sample_rows(logits.to(DEV), _words(rows), out)
    out = out.tolist()
    assert out[0] == 20 and out[1] == 20 and out[3] == 0
    assert out[2] == 7


def test_sample_rows_frequencies():
    """Many draws from one row: observed frequencies match the softmax."""
    V, n = 50, 4000
    g = torch.Generator().manual_seed(1)
    row = torch.randn(V, generator=g) * 2
    us = torch.rand(n, generator=g)
    rows = [(float(u), 1.0, 0, 1.0) for u in us]
    out = torch.zeros(n, dtype=torch.int32, device=DEV)
    kernels().sample_rows(row.repeat(n, 1).to(DEV), _words(rows), out)
    freq = torch.bincount(out.cpu().long(), minlength=V).double() / n
    p = torch.softmax(row.double(), 0)
    assert (freq - p).abs().max() < 4 * (p * (1 - p) / n).sqrt().max() + 1e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [1, 8, 20, 50, 100])
@pytest.mark.parametrize("n_heads,n_kv,hd,rot,K", [(4, 2, 32, 32, 256), (8, 2, 128, 128, 512), (3, 1, 64, 32, 96), (2, 2, 16, 0, 64),
                                                  (36, 2, 128, 128, 8192),     # long rows: at 50 tokens the product takes the tiles, the rotation its own kernel
                                                  (32, 8, 128, 128, 2048)])    # 6144 features: blocks of a tile and a half at 1 to 64 tokens
def test_qkv_rope_cache(dtype, M, n_heads, n_kv, hd, rot, K):
    """The product, the rotation by neighbouring pairs and the cache write, as one call: for a few
    bfloat16 tokens it is one kernel that rotates the 32-bit sums; else product, then rotation."""
    page_size, num_pages = 16, 12
    N = (n_heads + 2 * n_kv) * hd
    x = rnd((M, K), dtype, 30)
    w = rnd((N, K), dtype, 31, 0.1)
    positions = torch.randint(0, 400, (M,), generator=torch.Generator().manual_seed(32)).to(torch.int32).to(DEV)
    slots = torch.randperm(num_pages * page_size, generator=torch.Generator().manual_seed(33))[:M].to(torch.int32).to(DEV)
    inv_freq = plain_inv_freq(rot, 10000.0, None).to(DEV) if rot else None
    qkv = torch.zeros((M, N + 8), dtype=dtype, device=DEV)
    kc = torch.zeros((num_pages, n_kv, page_size, hd), dtype=dtype, device=DEV)
    vc = torch.zeros((num_pages, n_kv, hd, page_size), dtype=dtype, device=DEV)
    kernels().qkv_rope_cache(x, w, qkv[:, :N], positions, slots, inv_freq, rot, kc, vc, n_heads, n_kv, hd,
                             page_size, num_pages, True)
    acc = x.double().cpu() @ w.double().cpu().T
    q = acc[:, :n_heads * hd].view(M, n_heads, hd)
    k = acc[:, n_heads * hd:(n_heads + n_kv) * hd].view(M, n_kv, hd)
    v = acc[:, (n_heads + n_kv) * hd:].view(M, n_kv, hd)
    if rot:
        q = plain_rope(q, positions.cpu(), inv_freq.cpu(), "interleaved")
        k = plain_rope(k, positions.cpu(), inv_freq.cpu(), "interleaved")
    floor = 2e-6 * math.sqrt(K) if dtype == torch.float32 else 2e-2
    page, off = (slots // page_size).long().cpu(), (slots % page_size).long().cpu()
    got_q = qkv[:, :n_heads * hd].double().cpu().view(M, n_heads, hd)
    got_k = kc.double().cpu()[page, :, off, :]
    got_v = vc.double().cpu()[page, :, :, off]
    rel = 1.0 / 40 if dtype == torch.bfloat16 else 1e-5       # bfloat16 may round twice (product, then rotation)
    for name, got, ref in (("q", got_q, q), ("k", got_k, k), ("v", got_v, v)):
        err = (got - ref).abs()
        # a rotated value carries the rounding of both values of its pair, whose size is the pair's norm
        # (which the rotation keeps): what matters once the sums are large (K in the thousands)
        size = ref.abs()
        if rot and name != "v":
            pair = ref[..., :rot].unflatten(-1, (rot // 2, 2)).norm(dim=-1, keepdim=True).expand(-1, -1, -1, 2).flatten(-2)
            size = torch.cat([pair, size[..., rot:]], dim=-1)
        assert (err <= size * rel + floor).all(), f"{name}: max err {float(err.max())}"
    assert (qkv[:, N:] == 0).all(), "padding touched"


@pytest.mark.parametrize("M,n_heads,n_kv,hd,rot,K", [(100, 32, 8, 128, 128, 4096), (300, 16, 4, 64, 64, 2048), (64, 36, 2, 128, 128, 8192),
                                                    (200, 8, 8, 128, 64, 2048), (512, 32, 8, 64, 64, 2048), (65, 32, 8, 128, 128, 4096)])
def test_qkv_rope_cache_adds_up_a_split_product(M, n_heads, n_kv, hd, rot, K):
    """With 65 to 512 rows (and long rows from 33 on) the product is split over blocks along k and leaves the parts
    of its sums; the rotation kernel adds them up as it reads its rows.  The first 48 tokens fill three pages in
    order (their values are written page-wise, through LDS), the rest lie scattered."""
    page_size, num_pages = 16, 40
    N = (n_heads + 2 * n_kv) * hd
    k = kernels()
    n_ws = k.gemm_workspace_floats(M, N, K)
    assert n_ws >= 2 * M * N, "the case itself: a product that is split"
    x = rnd((M, K), torch.bfloat16, 30)
    w = rnd((N, K), torch.bfloat16, 31, 0.1)
    positions = torch.randint(0, 400, (M,), generator=torch.Generator().manual_seed(32)).to(torch.int32).to(DEV)
    pages = torch.randperm(num_pages, generator=torch.Generator().manual_seed(33)).tolist()
    in_order = [pages[i] * 16 + j for i in range(3) for j in range(16)]
    rest = [pg * 16 + j for pg in pages[3:] for j in range(16)]
    rest = [rest[i] for i in torch.randperm(len(rest), generator=torch.Generator().manual_seed(34)).tolist()]
    slots = torch.tensor((in_order + rest)[:M], dtype=torch.int32, device=DEV)
    inv_freq = plain_inv_freq(rot, 10000.0, None).to(DEV)
    qkv = torch.zeros((M, N + 8), dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros((num_pages, n_kv, page_size, hd), dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros((num_pages, n_kv, hd, page_size), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(n_ws, dtype=torch.float32, device=DEV)
    k.qkv_rope_cache(x, w, qkv[:, :N], positions, slots, inv_freq, rot, kc, vc, n_heads, n_kv, hd, page_size, num_pages, True, ws)
    acc = x.double().cpu() @ w.double().cpu().T
    q = plain_rope(acc[:, :n_heads * hd].view(M, n_heads, hd), positions.cpu(), inv_freq.cpu(), "interleaved")
    kk = plain_rope(acc[:, n_heads * hd:(n_heads + n_kv) * hd].view(M, n_kv, hd), positions.cpu(), inv_freq.cpu(), "interleaved")
    v = acc[:, (n_heads + n_kv) * hd:].view(M, n_kv, hd)
    page, off = (slots // page_size).long().cpu(), (slots % page_size).long().cpu()
    got_q = qkv[:, :n_heads * hd].double().cpu().view(M, n_heads, hd)
    got_k = kc.double().cpu()[page, :, off, :]
    got_v = vc.double().cpu()[page, :, :, off]
    for name, got, ref in (("q", got_q, q), ("k", got_k, kk), ("v", got_v, v)):
        err = (got - ref).abs()
        size = ref.abs()
        if name != "v":
            pair = ref[..., :rot].unflatten(-1, (rot // 2, 2)).norm(dim=-1, keepdim=True).expand(-1, -1, -1, 2).flatten(-2)
            size = torch.cat([pair, size[..., rot:]], dim=-1)
        assert (err <= size / 40 + 2e-2).all(), f"{name}: max err {float(err.max())}"
    assert (qkv[:, N:] == 0).all(), "padding touched"
    written = torch.zeros(num_pages * page_size, dtype=torch.bool)
    written[slots.long().cpu()] = True
    assert (kc.cpu().permute(0, 2, 1, 3).reshape(num_pages * page_size, -1)[~written] == 0).all(), "a slot that no token maps to was written"
    assert (vc.cpu().permute(0, 3, 1, 2).reshape(num_pages * page_size, -1)[~written] == 0).all(), "a slot that no token maps to was written"
    # the same call with room for nothing: product, then rotation, each a kernel of its own; the same results to rounding
    qkv2, kc2, vc2 = torch.zeros_like(qkv), torch.zeros_like(kc), torch.zeros_like(vc)
    k.qkv_rope_cache(x, w, qkv2[:, :N], positions, slots, inv_freq, rot, kc2, vc2, n_heads, n_kv, hd, page_size, num_pages, True)
    scale = float(acc.abs().max())
    assert (qkv2[:, :n_heads * hd].float() - qkv[:, :n_heads * hd].float()).abs().max() <= scale / 64
    assert (kc2.float() - kc.float()).abs().max() <= scale / 64 and (vc2.float() - vc.float()).abs().max() <= scale / 64


# ---- utilities ----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,key,mean,std", [(1, 5, 0.0, 0.02), (100003, 2**63 + 11, 1.0, 0.1), (3_000_001, 99, 0.0, 1.0)])
def test_seeded_fill_is_the_same_on_host_and_device(dtype, n, key, mean, std):
    """Random-weights mode makes a tensor where the engine lives; the plain implementation gets the
    host's.  They are the same function of (key, index), so they must agree in every bit."""
    from llm_rs_amd.weights import fill_normal
    host = fill_normal(torch.empty(n, dtype=dtype), key, mean, std)
    dev = fill_normal(torch.empty(n, dtype=dtype, device=DEV), key, mean, std)
    assert torch.equal(dev.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       host.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))


def test_random_model_is_the_same_on_host_and_device():
    from llm_rs_amd import LlamaConfig, random_model_tensors
    from tiny_configs import TINY_B
    cfg = LlamaConfig.from_dict(TINY_B)
    host, dev = random_model_tensors(cfg, 3), random_model_tensors(cfg, 3, device=DEV)
    assert sorted(host) == sorted(dev)
    for name in host:
        assert torch.equal(host[name], dev[name].cpu()), name


@pytest.mark.parametrize("src,dst", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                     (torch.float16, torch.bfloat16), (torch.float32, torch.float32)])
def test_cast(src, dst):
    x = rnd((7, 1001), torch.float32, 3, 5.0).to(src)
    out = torch.empty((7, 1001), dtype=dst, device=DEV)
    kernels().cast(out, x)
    assert torch.equal(out, x.to(dst))


def test_embed_rows_scaled():
    table = rnd((50, 72), torch.bfloat16, 0)
    tokens = torch.tensor([3, 49, 0], dtype=torch.int32, device=DEV)
    out = torch.empty((3, 72), dtype=torch.float32, device=DEV)
    kernels().embed_rows(out, table, tokens, 8.485281)
    assert torch.equal(out, table[tokens.long()].float() * torch.tensor(8.485281, dtype=torch.float32))


@pytest.mark.parametrize("scale,cap", [(0.25, 0.0), (1.0, 30.0), (0.5, 2.0)])
def test_scale_softcap_rows(scale, cap):
    x = rnd((5, 1003), torch.float32, 4, 20.0)
    big = x.clone()[:, :1000]                     # a view with a row stride, as logits of a padded buffer would be
    ref = big.double().cpu() * scale
    if cap > 0:
        ref = cap * torch.tanh(ref / cap)
    kernels().scale_softcap_rows(big, scale, cap)
    assert float((big.double().cpu() - ref).abs().max()) <= 1e-5 * max(1.0, float(ref.abs().max()))


# ---- a norm without a kernel of its own -----------------------------------------------------------

NORMED_SHAPES = [(8, 6144, 4096), (1, 6144, 4096), (1, 28672, 4096), (2, 28672, 4096), (8, 28672, 4096), (16, 28672, 4096),
                 (5, 16400, 256), (3, 8192, 16384), (16, 520, 128), (7, 200, 2048), (9, 4096, 14336), (4, 96, 72)]


def _left_for_norm(M, K, seed, weight):
    """A 32-bit stream and what the product that wrote it last leaves for the norm that follows: the rows times the
    norm's weight in bfloat16, and the sums of squares of each 16 features of a row."""
    h = rnd((M, K), torch.float32, seed, 2.0)
    parts = -(-K // 16)
    padded = torch.zeros((M, parts * 16), dtype=torch.float32, device=DEV)
    padded[:, :K] = h
    y = torch.zeros((M, K + 8), dtype=torch.bfloat16, device=DEV)[:, :K]        # rows with a stride
    y.copy_((h * weight).bfloat16())
    return h, y, (padded * padded).view(M, parts, 16).sum(-1).contiguous()


@pytest.mark.parametrize("epi", [EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU])
@pytest.mark.parametrize("M,N,K", NORMED_SHAPES)
def test_gemm_finishes_a_norm_left_to_it(M, N, K, epi):
    """x W^T with x = h inv weight, computed as inv (h weight) W^T: against float64 on the same rounded rows (tight),
    and against RMSNorm rounded to bfloat16 and then multiplied (the same up to where the one rounding falls)."""
    from llm_rs_amd.kernels import NormedRows
    k = kernels()
    assert k.gemm_defers_norm(M, N, K)
    eps = 1e-5
    nw = rnd((K,), torch.float32, 41) * 0.1 + 1
    h, y, sums = _left_for_norm(M, K, 40, nw)
    w = rnd((N, K), torch.bfloat16, 42, 0.1)
    inv = 1.0 / torch.sqrt((h.double().cpu() ** 2).sum(-1, keepdim=True) / K + eps)
    acc = (y.double().cpu() @ w.double().cpu().T) * inv
    other = plain_rmsnorm(h.double().cpu(), nw.double().cpu(), eps).bfloat16().double() @ w.double().cpu().T
    floor = 1e-5 * math.sqrt(K)
    if epi == EPI_STORE:
        out, ref, odt = torch.zeros((M, N), dtype=torch.bfloat16, device=DEV), acc, torch.bfloat16
    elif epi == EPI_STORE_F32:
        out, ref, odt = torch.zeros((M, N), dtype=torch.float32, device=DEV), acc, torch.float32
    elif epi == EPI_ACCUM_F32:
        out = rnd((M, N), torch.float32, 5)
        ref, other, odt = out.double().cpu() + acc, out.double().cpu() + other, torch.float32
    else:
        out = torch.zeros((M, N // 2), dtype=torch.bfloat16, device=DEV)
        ref, other, odt = plain_silu(acc[:, 0::2]) * acc[:, 1::2], plain_silu(other[:, 0::2]) * other[:, 1::2], torch.bfloat16
        floor *= 1 + 0.1 * math.sqrt(K)
    k.gemm(NormedRows(y, sums, eps), w, out, epi)
    err = (out.double().cpu() - ref).abs()
    tol = out_tol(ref, odt, floor)
    assert (err <= tol).all(), f"max err {float(err.max())} at {int(err.argmax())}, tol there {float(tol.flatten()[err.argmax()])}"
    # Where the one rounding falls: both ways round every input (of size 1) by up to 2^-9 of itself, independently,
    # (1.6e-3 of itself in standard deviation each), so an input differs by 2.3e-3 between them and a sum of K products
    # with weights of size 0.1 by 2.3e-3 * 0.1 * sqrt(K); six of those bound the largest of many outputs.  SwiGLU
    # multiplies a sum's deviation by the other sum, of size 0.1 sqrt(K).
    spread = 6 * 2.3e-3 * 0.1 * math.sqrt(K) * (2 * (1 + 0.1 * math.sqrt(K)) if epi == EPI_SWIGLU else 1)
    loose = out_tol(other, odt, floor + spread)
    assert ((out.double().cpu() - other).abs() <= loose).all()


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 4096, 14336), (16, 4096, 4096), (5, 200, 328), (3, 8192, 28672), (12, 100, 64),
                                   # narrow weights with long rows: blocks of 8 features, a partial sum for each
                                   (1, 2048, 8192), (8, 2048, 2048), (16, 1024, 4096), (3, 2040, 2048)])
def test_residual_product_leaves_what_the_next_norm_needs(M, N, K):
    from llm_rs_amd.kernels import NextNorm
    k = kernels()
    assert k.gemm_defers_norm(M, N, K)
    parts = k.gemm_next_parts(M, N, K)
    per = 16 if parts == -(-N // 16) else 8
    assert parts == -(-N // per) and (per == 8) == (N <= 2048 and K >= 2048)
    a = rnd((M, K), torch.bfloat16, 50)
    w = rnd((N, K), torch.bfloat16, 51, 0.1)
    h = rnd((M, N), torch.float32, 52, 2.0)
    nw = rnd((N,), torch.float32, 53) * 0.1 + 1
    want_h = h.double().cpu() + a.double().cpu() @ w.double().cpu().T
    sums = torch.full((M, parts), -1.0, dtype=torch.float32, device=DEV)
    y = torch.full((M, N + 4), 7.0, dtype=torch.bfloat16, device=DEV)
    plain = h.clone()
    k.gemm(a, w, plain, EPI_ACCUM_F32)
    k.gemm(a, w, h, EPI_ACCUM_F32, None, leave=NextNorm(y[:, :N], sums, nw))
    assert torch.equal(h, plain), "leaving something for the norm does not change the product"
    assert torch.equal(y[:, :N], (h * nw).bfloat16()) and (y[:, N:] == 7.0).all()
    padded = torch.zeros((M, parts * per), dtype=torch.float64)
    padded[:, :N] = h.double().cpu()
    want = (padded * padded).view(M, parts, per).sum(-1)
    assert float((sums.double().cpu() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    assert float((h.double().cpu() - want_h).abs().max()) <= 1e-5 * math.sqrt(K) + 1e-5 * float(want_h.abs().max())


@pytest.mark.parametrize("M,hidden,inter", [(1, 2048, 8192), (8, 2048, 8192), (16, 1024, 2048), (5, 4096, 14336), (3, 4096, 4096)])
def test_a_norm_left_by_one_product_and_finished_by_the_next(M, hidden, inter):
    """down -> (norm) -> q/k/v-like product, as a layer's end and the next layer's start: the second product's result
    against the norm kernel on the stream followed by the plain product.  Narrow streams leave a partial sum per 8
    features, the others per 16; the consumer takes whatever number of parts it is given."""
    from llm_rs_amd.kernels import NextNorm, NormedRows
    k = kernels()
    a = rnd((M, inter), torch.bfloat16, 80)
    w_down = rnd((hidden, inter), torch.bfloat16, 81, 0.05)
    w_next = rnd((3 * hidden // 2, hidden), torch.bfloat16, 82, 0.1)
    nw = rnd((hidden,), torch.float32, 83) * 0.1 + 1
    h = rnd((M, hidden), torch.float32, 84, 2.0)
    parts = k.gemm_next_parts(M, hidden, inter)
    left = NextNorm(torch.zeros((M, hidden), dtype=torch.bfloat16, device=DEV), torch.zeros((M, parts), device=DEV), nw)
    k.gemm(a, w_down, h, EPI_ACCUM_F32, None, leave=left)
    got = torch.zeros((M, w_next.shape[0]), dtype=torch.bfloat16, device=DEV)
    k.gemm(NormedRows(left.y, left.sumsq, 1e-5), w_next, got)
    x = torch.zeros((M, hidden), dtype=torch.bfloat16, device=DEV)
    k.rmsnorm(x, h, nw, 1e-5)
    want = torch.zeros_like(got)
    k.gemm(x, w_next, want)
    hd = h.double().cpu()
    exact = (hd / torch.sqrt((hd * hd).mean(-1, keepdim=True) + 1e-5) * nw.double().cpu()) @ w_next.double().cpu().T
    scale = float(exact.abs().max())
    assert float((got.double().cpu() - exact).abs().max()) <= 1.5 * float((want.double().cpu() - exact).abs().max()) + 2e-3 * scale
    assert float((got.double().cpu() - exact).abs().max()) <= 2e-2 * scale


@pytest.mark.parametrize("M,N,K", [(64, 4096, 4096), (17, 4096, 14336), (24, 1024, 2048), (33, 2048, 8192), (200, 512, 4096),
                                   (128, 4096, 4096), (256, 1000, 2048), (40, 6144, 4096), (64, 8192, 8192), (45, 4096, 4096),
                                   (2030, 2048, 2048), (1900, 2048, 8192), (700, 4096, 4096), (300, 1000, 2048)])
def test_split_residual_product_finishes_the_next_norm(M, N, K):
    """17 rows or more, a product whose sums are split over blocks: the kernel that adds the parts writes the stream and
    the normed rows: the stream bit for bit as without, the rows as the norm kernel makes them from that stream."""
    from llm_rs_amd.kernels import NextNorm
    k = kernels()
    assert k.gemm_norms_whole(M, N, K), "the case itself: this shape is split"
    a = rnd((M, K), torch.bfloat16, 70)
    w = rnd((N, K), torch.bfloat16, 71, 0.1)
    h = rnd((M, N), torch.float32, 72, 2.0)
    h[M // 2] *= 30.0               # one row far larger than the others: its scale must be its own
    nw = rnd((N,), torch.float32, 73) * 0.1 + 1
    eps = 3e-4
    ws = torch.empty(k.gemm_workspace_floats(M, N, K), dtype=torch.float32, device=DEV)
    plain = h.clone()
    k.gemm(a, w, plain, EPI_ACCUM_F32, ws)
    y = torch.full((M, N + 4), 7.0, dtype=torch.bfloat16, device=DEV)
    k.gemm(a, w, h, EPI_ACCUM_F32, ws, leave=NextNorm(y[:, :N], None, nw, eps))
    assert torch.equal(h, plain), "finishing the norm does not change the product"
    assert (y[:, N:] == 7.0).all(), "padding touched"
    want_h = rnd((M, N), torch.float32, 72, 2.0).double().cpu()
    want_h[M // 2] *= 30.0
    want_h += a.double().cpu() @ w.double().cpu().T
    assert float((h.double().cpu() - want_h).abs().max()) <= 1e-5 * math.sqrt(K) + 1e-5 * float(want_h.abs().max())
    normed = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    k.rmsnorm(normed, h, nw, eps)
    hd = h.double().cpu()
    exact = hd / torch.sqrt((hd * hd).mean(-1, keepdim=True) + eps) * nw.double().cpu()
    err = (y[:, :N].double().cpu() - exact).abs()
    assert (err <= exact.abs() * 2 ** -8 + 1e-6).all(), "within a rounding to bfloat16 of the exact norm"
    # the norm kernel adds the squares in another order: a unit in the last place here and there, no more
    differ = (y[:, :N].float() - normed.float()).abs()
    assert (differ <= normed.float().abs() * 2 ** -7 + 1e-6).all() and float((differ > 0).float().mean()) < 0.02


def test_a_norm_cannot_be_finished_by_a_product_that_is_not_split():
    from llm_rs_amd.kernels import KernelError, NextNorm
    k = kernels()
    M, N, K = 64, 24576, 4096
    assert not k.gemm_norms_whole(M, N, K)
    a, w = rnd((M, K), torch.bfloat16, 1), rnd((N, K), torch.bfloat16, 2, 0.1)
    h = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    y = torch.zeros((M, N), dtype=torch.bfloat16, device=DEV)
    with pytest.raises((KernelError, AssertionError)):
        k.gemm(a, w, h, EPI_ACCUM_F32, torch.empty(1 << 20, dtype=torch.float32, device=DEV), leave=NextNorm(y, None, torch.ones(N, device=DEV), 1e-5))


@pytest.mark.parametrize("M,n_heads,n_kv,hd,rot,K", [(8, 32, 8, 128, 128, 4096), (1, 32, 8, 128, 128, 4096), (16, 3, 1, 32, 32, 128),
                                                      (5, 4, 2, 16, 8, 64), (3, 64, 8, 128, 128, 8192), (7, 2, 2, 64, 0, 192)])
def test_qkv_rope_cache_finishes_a_norm_left_to_it(M, n_heads, n_kv, hd, rot, K):
    """Norm, product, rotation and cache write in one kernel, against the same call on the norm kernel's output."""
    from llm_rs_amd.kernels import NormedRows
    k = kernels()
    page_size, num_pages = 16, 12
    N = (n_heads + 2 * n_kv) * hd
    nw = rnd((K,), torch.float32, 61) * 0.1 + 1
    h, y, sums = _left_for_norm(M, K, 60, nw)
    w = rnd((N, K), torch.bfloat16, 62, 0.1)
    positions = torch.randint(0, 400, (M,), generator=torch.Generator().manual_seed(32)).to(torch.int32).to(DEV)
    slots = torch.randperm(num_pages * page_size, generator=torch.Generator().manual_seed(33))[:M].to(torch.int32).to(DEV)
    inv_freq = plain_inv_freq(rot, 10000.0, None).to(DEV) if rot else None
    results = []
    for fused in (True, False):
        qkv = torch.zeros((M, N + 8), dtype=torch.bfloat16, device=DEV)
        kc = torch.zeros((num_pages, n_kv, page_size, hd), dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros((num_pages, n_kv, hd, page_size), dtype=torch.bfloat16, device=DEV)
        if fused:
            x = NormedRows(y, sums, 1e-6)
        else:
            x = torch.empty((M, K), dtype=torch.bfloat16, device=DEV)
            k.rmsnorm(x, h, nw, 1e-6)
        k.qkv_rope_cache(x, w, qkv[:, :N], positions, slots, inv_freq, rot, kc, vc, n_heads, n_kv, hd, page_size, num_pages, True)
        results.append((qkv[:, :n_heads * hd].double().cpu(), kc.double().cpu(), vc.double().cpu()))
        assert (qkv[:, N:] == 0).all(), "padding touched"
    scale = max(float(results[1][0].abs().max()), 1.0)
    for name, a, b in zip("qkv", results[0], results[1]):
        # the two differ in where the one rounding of the rows falls
        assert float((a - b).abs().max()) <= 2e-2 * scale, name
        assert float((a - b).abs().mean()) <= 1.5e-3 * scale, name
