"""The kernels' plain C++ twins (llm_rs_amd/csrc/plain), called on CPU tensors through the same method names and
arguments as `llm_rs_amd.kernels.HipKernels`, so that a test can make one call on both.  Test equipment: the
package never loads the twins' library."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from llm_rs_amd.csrc.build import build_plain
from llm_rs_amd.kernels import EPI_ACCUM_F32, EPI_STORE, NextNorm, NormedRows

_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def _p(t: Optional[torch.Tensor]):
    if t is None:
        return None
    assert t.device.type == "cpu"
    return t.data_ptr()


class PlainTwins:
    def __init__(self):
        lib = ctypes.CDLL(build_plain())
        V, I, F, S = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
        sigs = {
            "llmrs_plain_embed_rows": [V, I, V, V, V, I, I, I, F],
            "llmrs_plain_rmsnorm": [V, I, V, V, V, V, I, I, F],
            "llmrs_plain_gemm": [V, I, V, I, V, V, I, I, I, I, I, V, S, I, V, I, F, V, V, I, V, F],
            "llmrs_plain_rope_kv_write": [V, I, V, I, V, V, V, I, I, V, V, I, I, I, I, I, I, I],
            "llmrs_plain_qkv_rope_cache": [V, I, V, I, V, V, I, I, I, V, V, V, I, V, V, I, I, I, I, I, I, V, S, I, V, I, F],
            "llmrs_plain_attention": [V, I, V, I, V, I, V, V, V, I, V, V, V, V, I, I, I, I, I, I, I, I, F, V, S, I, I, ctypes.c_long, I],
            "llmrs_plain_argmax_rows": [V, V, I, I, I, V, V, S],
            "llmrs_plain_sample_rows": [V, V, I, I, I, V, V, V],
            "llmrs_plain_place_ids": [V, V, I, V, V, V, I, I, I],
            "llmrs_plain_cast": [V, V, I, V, I, S],
            "llmrs_plain_scale_softcap_rows": [V, V, I, I, I, F, F],
        }
        for name, args in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = args, I
        self.lib = lib

    @staticmethod
    def _check(rc: int, what: str) -> None:
        if rc != 0:
            raise ValueError(f"the plain twin of {what} refused its arguments")

    def embed_rows(self, out, table, tokens, scale: float = 1.0) -> None:
        assert out.dtype == torch.float32 and tokens.dtype == torch.int32 and table.is_contiguous() and out.is_contiguous()
        self._check(self.lib.llmrs_plain_embed_rows(None, _CODE[table.dtype], _p(out), _p(table), _p(tokens), tokens.shape[0],
                                                    table.shape[1], table.shape[0], float(scale)), "embed_rows")

    def rmsnorm(self, out, x, weight, eps: float, rows=None) -> None:
        assert x.dtype == torch.float32 and weight.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous()
        self._check(self.lib.llmrs_plain_rmsnorm(None, _CODE[out.dtype], _p(out), _p(x), _p(weight), _p(rows), out.shape[0],
                                                 x.shape[1], float(eps)), "rmsnorm")

    def gemm(self, a, w, out, epilogue: int = EPI_STORE, workspace=None, leave: Optional[NextNorm] = None) -> None:
        scale = None
        if isinstance(a, NormedRows):
            scale, a = a, a.y
        M, K = a.shape
        whole = leave is not None and leave.whole
        assert leave is None or epilogue == EPI_ACCUM_F32
        self._check(self.lib.llmrs_plain_gemm(
            None, _CODE[a.dtype], _p(a), a.stride(0), _p(w), _p(out), out.stride(0), M, w.shape[0], K, epilogue, None, 0, 0,
            None if scale is None else _p(scale.sumsq), 0 if scale is None else scale.sumsq.shape[1],
            0.0 if scale is None else scale.eps, None if leave is None or whole else _p(leave.sumsq),
            None if leave is None else _p(leave.y), 0 if leave is None else leave.y.stride(0),
            None if leave is None else _p(leave.weight), leave.eps if whole else 0.0), "gemm")

    def rope_kv_write(self, qkv, positions, slot_map, inv_freq, rotary_dim, interleaved, k_cache, v_cache,
                      n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv) -> None:
        self._check(self.lib.llmrs_plain_rope_kv_write(
            None, _CODE[qkv.dtype], _p(qkv), qkv.stride(0), _p(positions), _p(slot_map), _p(inv_freq), rotary_dim,
            int(interleaved), _p(k_cache), _p(v_cache), qkv.shape[0], n_heads, n_kv_heads, head_dim, page_size, num_pages,
            int(write_kv)), "rope_kv_write")

    def qkv_rope_cache(self, x, w, qkv, positions, slot_map, inv_freq, rotary_dim, k_cache, v_cache,
                       n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv, workspace=None) -> None:
        scale = None
        if isinstance(x, NormedRows):
            scale, x = x, x.y
        self._check(self.lib.llmrs_plain_qkv_rope_cache(
            None, _CODE[x.dtype], _p(x), x.stride(0), _p(w), _p(qkv), qkv.stride(0), x.shape[0], x.shape[1], _p(positions),
            _p(slot_map), _p(inv_freq), rotary_dim, _p(k_cache), _p(v_cache), n_heads, n_kv_heads, head_dim, page_size,
            num_pages, int(write_kv), None, 0, 0, None if scale is None else _p(scale.sumsq),
            0 if scale is None else scale.sumsq.shape[1], 0.0 if scale is None else scale.eps), "qkv_rope_cache")

    def attention(self, q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, seq_lens,
                  n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale, scratch=None, max_seq_len=0,
                  n_single=-1, single_keys=0) -> None:
        self._check(self.lib.llmrs_plain_attention(
            None, _CODE[q.dtype], _p(q), q.stride(0), _p(out), out.stride(0), _p(k_cache), _p(v_cache), _p(block_table),
            block_table.shape[1], _p(token_entry), _p(positions), _p(q_starts), _p(seq_lens), block_table.shape[0],
            q.shape[0], n_heads, n_kv_heads, head_dim, page_size, num_pages, window, float(scale), None, 0, 0, 0, 0, 0),
            "attention")

    def argmax_rows(self, logits, out, scratch=None) -> None:
        self._check(self.lib.llmrs_plain_argmax_rows(None, _p(logits), logits.stride(0), logits.shape[0], logits.shape[1],
                                                     _p(out), None, 0), "argmax_rows")

    def sample_rows(self, logits, words, out, probs: Optional[torch.Tensor] = None) -> None:
        """probs (float64 [rows, V], optional): the probabilities each row was drawn from."""
        assert probs is None or (probs.dtype == torch.float64 and probs.is_contiguous() and probs.shape == logits.shape)
        self._check(self.lib.llmrs_plain_sample_rows(None, _p(logits), logits.stride(0), logits.shape[0], logits.shape[1],
                                                     _p(words), _p(out), _p(probs)), "sample_rows")

    def place_ids(self, tokens, rows, sources, ids, vocab: int) -> None:
        self._check(self.lib.llmrs_plain_place_ids(None, _p(tokens), tokens.numel(), _p(rows), _p(sources), _p(ids),
                                                   ids.numel(), rows.numel(), int(vocab)), "place_ids")

    def cast(self, dst, src) -> None:
        self._check(self.lib.llmrs_plain_cast(None, _p(dst), _CODE[dst.dtype], _p(src), _CODE[src.dtype], src.numel()), "cast")

    def scale_softcap_rows(self, logits, scale: float, cap: float) -> None:
        self._check(self.lib.llmrs_plain_scale_softcap_rows(None, _p(logits), logits.stride(0), logits.shape[0],
                                                            logits.shape[1], float(scale), float(cap)), "scale_softcap_rows")


_twins = None


def twins() -> PlainTwins:
    global _twins
    if _twins is None:
        _twins = PlainTwins()
    return _twins
