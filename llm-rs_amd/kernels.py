"""The kernel interface: every device operation of the engine goes through the
object `kernels()` returns.  It is the gfx950 library (csrc/hip) or nothing:
when that library cannot be built or loaded, or there is no GPU, the first use
raises.  `use_kernels()` lets a test put another object with the same methods in
its place; the package itself never does.

Op set of the reference's `Backend` trait (src/backend/mod.rs:15-89), fused:
embed, rms_norm, matmul (+ residual add / SwiGLU epilogues for add/silu/mul),
rope + scatter_kv, attention, gather (folded into rms_norm's row list), argmax.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import sys
from ctypes import c_char_p, c_float, c_int, c_size_t, c_void_p
from typing import Dict, List, NamedTuple, Optional

import torch

EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU = 0, 1, 2, 3
_EPI_NAMES = {EPI_STORE: "store", EPI_STORE_F32: "store32", EPI_ACCUM_F32: "add32", EPI_SWIGLU: "swiglu"}

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


# MI355X, published: HBM3E 8 TB/s; dense matrix cores 2.5 PFLOP/s in bfloat16, 157.3 TFLOP/s in float32
PEAK_HBM_BYTES = 8.0e12
PEAK_FLOPS = {torch.bfloat16: 2.5e15, torch.float32: 157.3e12}


class KernelError(RuntimeError):
    pass


class NormedRows:
    """Rows whose norm is left to the product that takes them (steps of a few tokens; no norm kernel runs).
    `y` [rows, K] holds the stream's rows times the norm's weight, rounded once to the activation type, and
    `sumsq` [rows, parts] the sums of squares of each 16 consecutive features of the stream's rows: both left
    by the product that added into the stream last.  The product multiplies each of its 32-bit sums by the row's
    1 / sqrt(sum(sumsq) / K + eps): x W^T with x = h inv weight equals inv (h weight) W^T."""

    def __init__(self, y: torch.Tensor, sumsq: torch.Tensor, eps: float):
        self.y, self.sumsq, self.eps = y, sumsq, float(eps)
        self.shape, self.dtype = y.shape, y.dtype


class NextNorm:
    """What a product that adds into the stream leaves for the norm that follows, see `NormedRows`:
    `y` and `sumsq` to fill, `weight` the following norm's.  With `eps` (and no `sumsq`) the product finishes the
    norm itself: `y` becomes the normed rows, for any product to take as they are (`gemm_norms_whole`: steps of
    17 tokens or more whose product is split over blocks, where the kernel that adds the parts up sees whole rows)."""

    def __init__(self, y: torch.Tensor, sumsq: Optional[torch.Tensor], weight: torch.Tensor, eps: float = 0.0):
        self.y, self.sumsq, self.weight, self.eps = y, sumsq, weight, float(eps)

    @property
    def whole(self) -> bool:
        return self.eps > 0.0


class KernelTimes:
    """Per-kernel device time with the bytes each call has to move and the operations it has to
    do, as the reference keeps when LLM_PERF is set (src/backend/metal/mod.rs:321-400): a pair of
    events around every call, read when the table is asked for."""

    def __init__(self):
        self.calls: List[tuple] = []       # (label, bytes, flops, peak flops, start event, end event)

    def add(self, label, nbytes, flops, peak, start, end):
        self.calls.append((label, nbytes, flops, peak, start, end))

    def rows(self) -> List[dict]:
        """One row per label, most device time first; clears what was recorded."""
        torch.cuda.synchronize()
        acc: Dict[str, dict] = {}
        for label, nbytes, flops, peak, start, end in self.calls:
            r = acc.setdefault(label, {"kernel": label, "calls": 0, "seconds": 0.0, "bytes": 0, "flops": 0, "peak_flops": peak})
            r["calls"] += 1
            r["seconds"] += start.elapsed_time(end) * 1e-3
            r["bytes"] += nbytes
            r["flops"] += flops
        self.calls = []
        rows = sorted(acc.values(), key=lambda r: -r["seconds"])
        for r in rows:
            t = max(r["seconds"], 1e-12)
            r["gb_per_s"] = r["bytes"] / t / 1e9
            r["hbm_frac"] = r["bytes"] / t / PEAK_HBM_BYTES
            r["tflops"] = r["flops"] / t / 1e12
            r["flops_frac"] = r["flops"] / t / r["peak_flops"] if r["peak_flops"] else 0.0
        return rows

    def dump(self, file=None) -> List[dict]:
        file = file or sys.stderr
        rows = self.rows()
        if not rows:
            return rows
        total = sum(r["seconds"] for r in rows)
        print(f"  {'kernel':<34} {'calls':>6} {'GPU time':>10} {'% total':>8}  {'GB/s (% of 8 TB/s)':>20}  {'TFLOP/s (% of peak)':>20}", file=file)
        print("  " + "-" * 106, file=file)
        for r in rows:
            t = f"{r['seconds'] * 1e3:.2f}ms" if r["seconds"] >= 1e-3 else f"{r['seconds'] * 1e6:.0f}us"
            fl = f"{r['tflops']:.1f} ({r['flops_frac'] * 100:.1f}%)" if r["flops"] else "-"
            print(f"  {r['kernel']:<34} {r['calls']:>6} {t:>10} {r['seconds'] / total * 100:>7.1f}%  "
                  f"{r['gb_per_s']:>10.0f} ({r['hbm_frac'] * 100:>4.1f}%)  {fl:>20}", file=file)
        all_bytes = sum(r["bytes"] for r in rows)
        print("  " + "-" * 106, file=file)
        print(f"  {'TOTAL':<34} {'':>6} {total * 1e3:>8.2f}ms {'100.0%':>8}  {all_bytes / total / 1e9:>10.0f} ({all_bytes / total / PEAK_HBM_BYTES * 100:>4.1f}%)",
              file=file)
        return rows


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class NormPlan(NamedTuple):
    """How a product that adds into the stream serves the norm that follows it (`Kernels.norm_left_by_product`)."""
    whole: bool          # True: the product finishes the norm itself (a `NextNorm` with eps, and the product's workspace)
    parts: int           # else: partial sums of squares it leaves per row, the second dimension of `NextNorm.sumsq`


class Kernels:
    """What the engine asks of its device operations beyond the operations themselves: how much room a call needs and
    which of the optional hand-overs between kernels a call can take.  An implementation answers for itself; the
    answers here are those of one that splits nothing and hands nothing over, so that parts never have to probe the
    object they were given."""

    allow_mfma = False
    times: Optional[KernelTimes] = None

    def gemm_workspace_floats(self, M: int, N: int, K: int) -> int:
        """Room (floats) that lets the product of M rows with an [N, K] weight split K over blocks; 0: none needed."""
        return 0

    def product_norms_its_rows(self, M: int, N: int, K: int, dtype: torch.dtype) -> bool:
        """Whether the product of M rows with an [N, K] weight takes `NormedRows` (rows still to be scaled by
        their norm) in place of normed rows."""
        return False

    def norm_left_by_product(self, M: int, N: int, K: int, dtype: torch.dtype) -> Optional[NormPlan]:
        """What the product of M rows with an [N, K] weight, adding into the stream, can leave for the norm that
        reads the stream next (`NextNorm`), or None: then a norm kernel runs."""
        return None

    def attention_scratch_floats(self, n_entries: int, n_heads: int, head_dim: int, max_seq_len: int,
                                 n_kv_heads: Optional[int] = None, n_single: int = 0) -> int:
        """Room (floats) for the partial results of single-token entries whose keys are shared out over waves."""
        return 0

    def attention_split_chunk(self, n_single: int, n_kv_heads: int, head_dim: int, max_seq_len: int, single_keys: int = 0) -> int:
        """Keys per wave that a call with these figures splits its single-token entries by (0: it does not split):
        what a caller that records steps has to key its recordings by."""
        return 0


class HipKernels(Kernels):
    """Launches on the current torch stream of the tensors' device."""

    def __init__(self):
        from .csrc.build import load_hip
        if not torch.cuda.is_available():
            raise KernelError("no GPU: the engine's kernels are gfx950 HIP kernels and there is no other path")
        self.lib = lib = load_hip()
        lib.llmrs_hip_error.restype = c_char_p
        V, I, F = c_void_p, c_int, c_float
        sigs = {
            "llmrs_embed_rows": [V, I, V, V, V, I, I, I, F],
            "llmrs_fill_normal": [V, I, V, c_size_t, ctypes.c_uint64, ctypes.c_uint64, F, F],
            "llmrs_cast": [V, V, I, V, I, c_size_t],
            "llmrs_scale_softcap_rows": [V, V, I, I, I, F, F],
            "llmrs_rmsnorm": [V, I, V, V, V, V, I, I, F],
            "llmrs_gemm": [V, I, V, I, V, V, I, I, I, I, I, V, c_size_t, I, V, I, F, V, V, I, V, F],
            "llmrs_gemm_defers_norm": [I, I, I],
            "llmrs_gemm_norms_whole": [I, I, I],
            "llmrs_gemm_next_parts": [I, I, I],
            "llmrs_rope_kv_write": [V, I, V, I, V, V, V, I, I, V, V, I, I, I, I, I, I, I],
            "llmrs_attention": [V, I, V, I, V, I, V, V, V, I, V, V, V, V, I, I, I, I, I, I, I, I, F, V, c_size_t, I, I, ctypes.c_long, I],
            "llmrs_qkv_rope_cache": [V, I, V, I, V, V, I, I, I, V, V, V, I, V, V, I, I, I, I, I, I, V, c_size_t, I, V, I, F],
            "llmrs_argmax_rows": [V, V, I, I, I, V, V, c_size_t],
            "llmrs_sample_rows": [V, V, I, I, I, V, V],
            "llmrs_place_ids": [V, V, I, V, V, V, I, I, I],
        }
        for name, args in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = I
        buf = ctypes.create_string_buffer(64)
        lib.llmrs_device_arch.argtypes = [c_char_p, I]
        lib.llmrs_device_arch.restype = I
        self.compute_units = lib.llmrs_device_arch(buf, 64)
        self.arch = buf.value.decode()
        if not self.arch.startswith("gfx950"):
            raise KernelError(f"the kernel library is built for gfx950, the device is {self.arch!r}")
        self.allow_mfma = True  # tests switch the matrix-core kernels off to compare paths
        # LLM_PERF in the environment (the reference's switch): every call is timed on the device and
        # steps are not recorded into graphs, so that each kernel can be seen by itself
        self.times: Optional[KernelTimes] = KernelTimes() if os.environ.get("LLM_PERF") else None
        lib.llmrs_attention_scratch_floats.restype = ctypes.c_long
        lib.llmrs_attention_scratch_floats.argtypes = [I, I, I, I, I, I]
        lib.llmrs_attention_split_chunk.restype = I
        lib.llmrs_attention_split_chunk.argtypes = [ctypes.c_long, I, I, I, ctypes.c_long]
        lib.llmrs_gemm_workspace_floats.restype = ctypes.c_long
        lib.llmrs_gemm_workspace_floats.argtypes = [I, I, I]

    def gemm_workspace_floats(self, M: int, N: int, K: int) -> int:
        """Room that lets a product with too few blocks split K over blocks (the kernels' own rule)."""
        return int(self.lib.llmrs_gemm_workspace_floats(int(M), int(N), int(K)))

    def product_norms_its_rows(self, M: int, N: int, K: int, dtype: torch.dtype) -> bool:
        return dtype == torch.bfloat16 and self.gemm_defers_norm(M, N, K)

    def norm_left_by_product(self, M: int, N: int, K: int, dtype: torch.dtype) -> Optional[NormPlan]:
        if dtype != torch.bfloat16:
            return None
        # up to a few rows: partial sums of squares, for the next product to finish (the kernels keep at most 1024
        # of them a row); more rows: a product that is split over blocks finishes the norm where its parts are added up
        if N < 16384 and self.gemm_defers_norm(M, N, K):
            return NormPlan(False, self.gemm_next_parts(M, N, K))
        if self.gemm_norms_whole(M, N, K):
            return NormPlan(True, 0)
        return None

    def gemm_defers_norm(self, M: int, N: int, K: int) -> bool:
        """Whether the bfloat16 product of M rows with an [N, K] weight takes `NormedRows` as its rows and, adding
        into the stream, leaves a `NextNorm` (that: for fewer than 16384 features)."""
        return self.allow_mfma and bool(self.lib.llmrs_gemm_defers_norm(int(M), int(N), int(K)))

    def gemm_next_parts(self, M: int, N: int, K: int) -> int:
        """Partial sums of squares per row that a product leaving a `NextNorm` writes (one per 16 features, for some
        shapes per 8): the second dimension of `NextNorm.sumsq`."""
        return int(self.lib.llmrs_gemm_next_parts(int(M), int(N), int(K)))

    def gemm_norms_whole(self, M: int, N: int, K: int) -> bool:
        """Whether the bfloat16 product of M rows with an [N, K] weight, adding into the stream with the workspace
        `gemm_workspace_floats` asks for, can finish the norm that follows (a `NextNorm` with eps)."""
        return self.allow_mfma and bool(self.lib.llmrs_gemm_norms_whole(int(M), int(N), int(K)))

    def attention_scratch_floats(self, n_entries: int, n_heads: int, head_dim: int, max_seq_len: int,
                                 n_kv_heads: Optional[int] = None, n_single: int = 0) -> int:
        """Room the split of single-token entries needs for its partial results (the kernels' own rule: the key
        ranges get shorter when there are few such entries)."""
        return int(self.lib.llmrs_attention_scratch_floats(int(n_entries), int(n_single), int(n_heads),
                                                            int(n_kv_heads or n_heads), int(head_dim), int(max_seq_len)))

    def _check(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.lib.llmrs_hip_error().decode())

    def _run(self, label: str, nbytes: int, flops: int, dtype, fn, *args) -> None:
        """Calls the library; with timing on, between two events, noting what the call has to move and to compute."""
        if self.times is None:
            return self._check(fn(*args))
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        self._check(fn(*args))
        end.record()
        self.times.add(label, int(nbytes), int(flops), PEAK_FLOPS.get(dtype, 0.0), start, end)

    @staticmethod
    def _stream() -> int:
        return torch.cuda.current_stream().cuda_stream

    # out[t, :] = table[tokens[t], :] * scale as float32
    def embed_rows(self, out: torch.Tensor, table: torch.Tensor, tokens: torch.Tensor, scale: float = 1.0) -> None:
        assert out.dtype == torch.float32 and tokens.dtype == torch.int32 and table.is_contiguous() and out.is_contiguous()
        assert out.shape[0] == tokens.shape[0] and out.shape[1] == table.shape[1]
        self._run("embed", out.numel() * (4 + table.element_size()), 0, None,
                  self.lib.llmrs_embed_rows, self._stream(), _code(table.dtype), _p(out), _p(table), _p(tokens),
                  tokens.shape[0], table.shape[1], table.shape[0], float(scale))

    # out.flat[i] = mean + std * normal(seed, first + i): the same bits as the host library makes
    def fill_normal(self, out: torch.Tensor, seed: int, mean: float, std: float, first: int = 0) -> None:
        assert out.is_contiguous()
        self._check(self.lib.llmrs_fill_normal(self._stream(), _code(out.dtype), _p(out), out.numel(), seed & (2**64 - 1),
                                               int(first), float(mean), float(std)))

    # dst = src in dst's dtype (float32, bfloat16; src may be float16 too), both on the device
    def cast(self, dst: torch.Tensor, src: torch.Tensor) -> None:
        codes = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
        assert dst.is_contiguous() and src.is_contiguous() and dst.numel() == src.numel()
        if dst.dtype not in (torch.float32, torch.bfloat16) or src.dtype not in codes:
            raise KernelError(f"no cast from {src.dtype} to {dst.dtype}")
        self._check(self.lib.llmrs_cast(self._stream(), _p(dst), codes[dst.dtype], _p(src), codes[src.dtype], src.numel()))

    # logits <- logits * scale, then cap * tanh(logits / cap) if cap > 0, in place
    def scale_softcap_rows(self, logits: torch.Tensor, scale: float, cap: float) -> None:
        assert logits.dtype == torch.float32 and logits.stride(1) == 1
        self._check(self.lib.llmrs_scale_softcap_rows(self._stream(), _p(logits), logits.stride(0), logits.shape[0],
                                                      logits.shape[1], float(scale), float(cap)))

    # out[i, :] = rmsnorm(x[rows[i] or i, :]) * weight
    def rmsnorm(self, out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float,
                rows: Optional[torch.Tensor] = None) -> None:
        assert x.dtype == torch.float32 and weight.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous()
        n = out.shape[0]
        assert out.shape[1] == x.shape[1] == weight.shape[0]
        assert (rows is None and n == x.shape[0]) or (rows is not None and rows.dtype == torch.int32 and rows.shape[0] == n)
        self._run(f"rmsnorm {n}x{x.shape[1]}", n * x.shape[1] * (4 + out.element_size()) + x.shape[1] * 4, 5 * n * x.shape[1], None,
                  self.lib.llmrs_rmsnorm, self._stream(), _code(out.dtype), _p(out), _p(x), _p(weight), _p(rows),
                  n, x.shape[1], eps)

    # out (epilogue) a @ w.T ; a: [M, K] rows may be strided, w: [N, K] dense
    def gemm(self, a, w: torch.Tensor, out: torch.Tensor, epilogue: int = EPI_STORE,
             workspace: Optional[torch.Tensor] = None, leave: Optional[NextNorm] = None) -> None:
        """`a` may be `NormedRows`, and `leave` a `NextNorm` (with the += epilogue), where `gemm_defers_norm` holds."""
        scale = None
        if isinstance(a, NormedRows):
            scale, a = a, a.y
            assert scale.sumsq.dtype == torch.float32 and scale.sumsq.is_contiguous() and scale.sumsq.shape[0] == a.shape[0]
        M, K = a.shape
        N = w.shape[0]
        assert w.shape[1] == K and w.is_contiguous() and a.stride(1) == 1 and out.stride(1) == 1 and a.dtype == w.dtype
        whole = leave is not None and leave.whole
        if leave is not None:
            assert epilogue == EPI_ACCUM_F32 and tuple(leave.y.shape) == (M, N) and leave.y.stride(1) == 1
            assert leave.y.dtype == torch.bfloat16 and leave.weight.dtype == torch.float32 and leave.weight.shape[0] == N
            if not whole:
                assert N < 16384 and leave.sumsq.dtype == torch.float32 and leave.sumsq.is_contiguous()
                assert tuple(leave.sumsq.shape) == (M, self.gemm_next_parts(M, N, K))
        if whole:
            assert a.dtype == torch.bfloat16 and scale is None and self.gemm_norms_whole(M, N, K) and workspace is not None
        elif scale is not None or leave is not None:
            assert a.dtype == torch.bfloat16 and self.gemm_defers_norm(M, N, K)
        want = torch.float32 if epilogue in (EPI_STORE_F32, EPI_ACCUM_F32) else a.dtype
        assert out.dtype == want and out.shape[0] == M and out.shape[1] == (N // 2 if epilogue == EPI_SWIGLU else N)
        moved = (M * K + N * K) * a.element_size() + out.numel() * out.element_size() * (2 if epilogue == EPI_ACCUM_F32 else 1)
        label = f"gemm {M}x{N}x{K} {'norm+' if scale is not None else ''}{_EPI_NAMES[epilogue]}{('+norm' if whole else '+next') if leave is not None else ''}"
        self._run(label, moved, 2 * M * N * K, a.dtype,
                  self.lib.llmrs_gemm, self._stream(), _code(a.dtype), _p(a), a.stride(0), _p(w), _p(out), out.stride(0),
                  M, N, K, epilogue, _p(workspace),
                  0 if workspace is None else workspace.numel() * workspace.element_size(), int(self.allow_mfma),
                  None if scale is None else _p(scale.sumsq), 0 if scale is None else scale.sumsq.shape[1],
                  0.0 if scale is None else scale.eps, None if leave is None or whole else _p(leave.sumsq),
                  None if leave is None else _p(leave.y), 0 if leave is None else leave.y.stride(0),
                  None if leave is None else _p(leave.weight), leave.eps if whole else 0.0)

    def rope_kv_write(self, qkv, positions, slot_map, inv_freq, rotary_dim, interleaved, k_cache, v_cache,
                      n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv) -> None:
        assert qkv.stride(1) == 1 and positions.dtype == torch.int32
        assert rotary_dim == 0 or (inv_freq.dtype == torch.float32 and inv_freq.shape[0] == rotary_dim // 2)
        if write_kv:
            assert k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
            assert k_cache.numel() == num_pages * n_kv_heads * page_size * head_dim == v_cache.numel()
            assert slot_map.dtype == torch.int32 and slot_map.shape[0] == qkv.shape[0]
        T = qkv.shape[0]
        self._run("rope_kv_write", T * (2 * n_heads + 4 * n_kv_heads) * head_dim * qkv.element_size(),
                  5 * T * (n_heads + n_kv_heads) * rotary_dim, None, self.lib.llmrs_rope_kv_write,
                  self._stream(), _code(qkv.dtype), _p(qkv), qkv.stride(0), _p(positions), _p(slot_map), _p(inv_freq),
                  rotary_dim, int(interleaved), _p(k_cache), _p(v_cache), qkv.shape[0], n_heads, n_kv_heads, head_dim,
                  page_size, num_pages, int(write_kv))

    def qkv_rope_cache(self, x, w, qkv, positions, slot_map, inv_freq, rotary_dim, k_cache, v_cache,
                       n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv, workspace=None) -> None:
        """qkv = x @ w.T, q and k rotated by adjacent pairs (2i, 2i+1), k and v written to the cache: fused into
        one kernel where the product allows.  Afterwards only the q part of `qkv` is certain to be filled."""
        assert w.shape[0] == (n_heads + 2 * n_kv_heads) * head_dim and w.shape[1] == x.shape[1] and qkv.shape[0] == x.shape[0]
        scale = None
        if isinstance(x, NormedRows):
            scale, x = x, x.y
            assert scale.sumsq.dtype == torch.float32 and scale.sumsq.is_contiguous() and scale.sumsq.shape[0] == x.shape[0]
            assert x.dtype == torch.bfloat16 and self.gemm_defers_norm(x.shape[0], w.shape[0], x.shape[1])
        assert x.stride(1) == 1 and qkv.stride(1) == 1 and w.is_contiguous() and x.dtype == w.dtype == qkv.dtype
        assert rotary_dim == 0 or (inv_freq.dtype == torch.float32 and inv_freq.shape[0] == rotary_dim // 2)
        if write_kv:
            assert k_cache.dtype == x.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
            assert k_cache.numel() == num_pages * n_kv_heads * page_size * head_dim == v_cache.numel()
        M, K, N = x.shape[0], x.shape[1], w.shape[0]
        self._run(f"gemm {M}x{N}x{K} {'norm+' if scale is not None else ''}qkv+rope+cache", (M * K + N * K + M * N) * x.element_size(), 2 * M * N * K, x.dtype,
                  self.lib.llmrs_qkv_rope_cache,
                  self._stream(), _code(x.dtype), _p(x), x.stride(0), _p(w), _p(qkv), qkv.stride(0), x.shape[0], x.shape[1],
                  _p(positions), _p(slot_map), _p(inv_freq), rotary_dim, _p(k_cache), _p(v_cache), n_heads, n_kv_heads,
                        head_dim, page_size, num_pages, int(write_kv), _p(workspace),
                  0 if workspace is None else workspace.numel() * workspace.element_size(), int(self.allow_mfma),
                  None if scale is None else _p(scale.sumsq), 0 if scale is None else scale.sumsq.shape[1],
                  0.0 if scale is None else scale.eps)

    def attention_split_chunk(self, n_single: int, n_kv_heads: int, head_dim: int, max_seq_len: int, single_keys: int = 0) -> int:
        """Keys per wave that a call with these figures splits its single-token entries by: what a caller that
        records steps into graphs has to key its recordings by, since a recording holds the chunk it was made with
        while the number of keys moves with every step."""
        return int(self.lib.llmrs_attention_split_chunk(int(n_single), int(n_kv_heads), int(head_dim), int(max_seq_len), int(single_keys)))

    def attention(self, q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, seq_lens,
                  n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale, scratch=None, max_seq_len=0, n_single=-1,
                  single_keys=0) -> None:
        """single_keys: how many keys the single-token entries see together (windows counted), 0 if unknown."""
        assert q.stride(1) == 1 and out.stride(1) == 1 and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype
        assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
        assert k_cache.numel() == num_pages * n_kv_heads * page_size * head_dim == v_cache.numel()
        T = q.shape[0]
        assert token_entry.shape[0] == T and positions.shape[0] == T and out.shape[0] == T
        moved = flops = 0
        if self.times is not None:      # what the call has to read depends on the step: ask the device (timing mode only)
            keys = int(seq_lens.sum().item())
            seen = int((positions + 1).sum().item()) if window <= 0 else int((positions + 1).clamp(max=window).sum().item())
            moved = (2 * keys * n_kv_heads + 2 * T * n_heads) * head_dim * q.element_size()
            flops = 4 * seen * n_heads * head_dim
        self._run(f"attention {T} tokens" + (" (decode)" if n_single == block_table.shape[0] else ""), moved, flops, q.dtype,
                  self.lib.llmrs_attention,
                  self._stream(), _code(q.dtype), _p(q), q.stride(0), _p(out), out.stride(0), _p(k_cache), _p(v_cache),
                  _p(block_table), block_table.shape[1], _p(token_entry), _p(positions), _p(q_starts), _p(seq_lens),
                  block_table.shape[0], T, n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale,
                  _p(scratch), 0 if scratch is None else scratch.numel() * scratch.element_size(), int(max_seq_len),
                  int(n_single), int(single_keys), int(self.allow_mfma))

    def argmax_rows(self, logits: torch.Tensor, out: torch.Tensor, scratch: Optional[torch.Tensor] = None) -> None:
        """`scratch`: 256 bytes per row let several blocks share a long row."""
        assert logits.dtype == torch.float32 and logits.stride(1) == 1 and out.dtype == torch.int32
        self._run("argmax", logits.numel() * 4, 0, None,
                  self.lib.llmrs_argmax_rows, self._stream(), _p(logits), logits.stride(0), logits.shape[0],
                  logits.shape[1], _p(out), _p(scratch), 0 if scratch is None else scratch.numel() * scratch.element_size())

    def place_ids(self, tokens: torch.Tensor, rows: torch.Tensor, sources: torch.Tensor, ids: torch.Tensor, vocab: int) -> None:
        """tokens[rows[i]] = ids[sources[i]]: what a step sampled goes into the next step's tokens on the device."""
        assert all(t.dtype == torch.int32 and t.is_contiguous() for t in (tokens, rows, sources, ids)) and rows.numel() == sources.numel()
        self._run("place_ids", rows.numel() * 12, 0, None,
                  self.lib.llmrs_place_ids, self._stream(), _p(tokens), tokens.numel(), _p(rows), _p(sources), _p(ids),
                  ids.numel(), rows.numel(), int(vocab))

    # words[i] = uniform (float bits), temperature (float bits), top_k, top_p (float bits) of row i
    def sample_rows(self, logits: torch.Tensor, words: torch.Tensor, out: torch.Tensor) -> None:
        assert logits.dtype == torch.float32 and logits.stride(1) == 1 and out.dtype == torch.int32
        assert words.dtype == torch.int32 and words.is_contiguous() and words.shape == (logits.shape[0], 4)
        self._run("sample", logits.numel() * 4, 0, None,
                  self.lib.llmrs_sample_rows, self._stream(), _p(logits), logits.stride(0), logits.shape[0],
                  logits.shape[1], _p(words), _p(out))


_kernels = None


def kernels():
    global _kernels
    if _kernels is None:
        _kernels = HipKernels()
    return _kernels


@contextlib.contextmanager
def use_kernels(obj):
    """For tests: run the engine's host logic against a stand-in for the device."""
    global _kernels
    old, _kernels = _kernels, obj
    try:
        yield obj
    finally:
        _kernels = old
