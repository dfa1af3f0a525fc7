"""Causal grouped-query attention over the paged cache.

Parameters: hidden_size, num_heads, num_kv_heads, head_dim, window (None: every
earlier key), position (a position-encoding spec or None), scale (None:
1/sqrt(head_dim), shaders/ops.metal:670), kv_proj (False: the part has no k and
v of its own and only reads a cache that another run wrote).

One step (src/arch/llama.rs:153-163): q, k, v = x Wq^T, x Wk^T, x Wv^T in one
product over the row-concatenated weight; q and k rotated and k, v written into
their pages by the same kernel (for a few tokens) or the next; attention of
every query token over its request's pages; h += o Wo^T with the sum fused into
the product.  No biases.

The rotation kernels pair neighbours (2i, 2i+1).  Where the encoding pairs
(i, i + rotary_dim/2), the rows of Wq and Wk are reordered within each head at
load so that those two features become neighbours: q.k is a sum over features
and does not care in which order q and k list them, as long as it is the same;
the reference runs files converted for exactly this order (src/arch/llama.rs:156).
"""
from __future__ import annotations

import math

import torch

from ..cache.spec import PagedKV
from ..kernels import EPI_ACCUM_F32, EPI_STORE, kernels
from .base import Mixer, TensorSpec, build_position, place, register_mixer


class Attention(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.window = int(p.get("window") or 0)
        self.recording_signature = ("attention", self.kv_heads, self.head_dim, self.window)
        self.kv_proj = bool(p.get("kv_proj", True))
        scale = p.get("scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.position = build_position(p.get("position"), dtype)
        if self.position is not None and self.position.rotary() is None:
            self.graph_safe = False      # its apply() is free to do anything
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are no multiple of {self.kv_heads} kv heads")
        self.q_size = self.heads * self.head_dim
        self.kv_size = self.kv_heads * self.head_dim
        self.w_qkv = None
        self.w_o = None

    def tensors(self):
        t = {self.name("q_proj.weight"): TensorSpec((self.q_size, self.hidden)),
             self.name("o_proj.weight"): TensorSpec((self.hidden, self.q_size))}
        if self.kv_proj:
            t[self.name("k_proj.weight")] = TensorSpec((self.kv_size, self.hidden))
            t[self.name("v_proj.weight")] = TensorSpec((self.kv_size, self.hidden))
        return t

    def _pair_neighbours(self, w: torch.Tensor, heads: int, undo: bool = False) -> torch.Tensor:
        """Rows of a q or k weight reordered so that each rotation pair is (2i, 2i+1); `undo` puts them back."""
        rotary = self.position.rotary() if self.position is not None else None
        if rotary is None or rotary[2] or rotary[1] == 0:
            return w          # no rotation here, or the pairs are neighbours already
        rot = rotary[1]
        order = torch.stack([torch.arange(rot // 2), torch.arange(rot // 2) + rot // 2], dim=1).flatten()
        order = torch.cat([order, torch.arange(rot, self.head_dim)])
        if undo:
            order = torch.argsort(order)
        return w.view(heads, self.head_dim, -1)[:, order.to(w.device), :].reshape(w.shape)

    def load(self, tensors, device):
        get = lambda n: place(tensors[self.name(n)], device, self.dtype)
        parts = [self._pair_neighbours(get("q_proj.weight"), self.heads)]
        if self.kv_proj:
            parts += [self._pair_neighbours(get("k_proj.weight"), self.kv_heads), get("v_proj.weight")]
        self.w_qkv = torch.cat(parts, dim=0).contiguous()
        self.w_o = get("o_proj.weight")
        if self.position is not None:
            self.position.to(device)

    def export(self):
        w = self.w_qkv.cpu()
        out = {self.name("q_proj.weight"): self._pair_neighbours(w[:self.q_size], self.heads, undo=True).contiguous(),
               self.name("o_proj.weight"): self.w_o.cpu()}
        if self.kv_proj:
            k, v = w[self.q_size:self.q_size + self.kv_size], w[self.q_size + self.kv_size:]
            out[self.name("k_proj.weight")] = self._pair_neighbours(k, self.kv_heads, undo=True).contiguous()
            out[self.name("v_proj.weight")] = v.contiguous()
        return out

    def cache_need(self):
        return PagedKV(self.kv_heads, self.head_dim, self.window)

    def takes_normed_rows(self, ctx, rows):
        # the q/k/v product norms its rows itself where it is the fused kernel: a rotation it applies (or none)
        fused = self.position is None or self.position.rotary() is not None
        return fused and kernels().product_norms_its_rows(rows, self.w_qkv.shape[0], self.hidden, self.dtype)

    # The kernel library shares the decoding requests' keys out over waves in chunks whose length it chooses by
    # how many keys the step sees (`single_keys`).  A recorded step holds the chunk it was recorded with, so the
    # chunk is part of what recordings are keyed by; and since recording a step again costs about as much as a step
    # while a chunk that is no longer the best one costs a few per cent of the attention, a batch keeps the figure
    # it was recorded with until the rule has asked for another chunk this many steps in a row.
    chunk_patience = 256

    def recording_key(self, ctx):
        k = kernels()
        if not ctx.n_single:
            return 0
        keys = ctx.single_keys(self.window)
        want = k.attention_split_chunk(ctx.n_single, self.kv_heads, self.head_dim, ctx.max_seq_len, keys)
        held = ctx.part_state.setdefault(self.recording_signature, {})
        at = (ctx.n_single, ctx.max_seq_len)
        now = held.get(at)             # [chunk, a number of keys that gives it, steps in a row that wanted another, step]
        if now is None or want == now[0] or now[2] >= self.chunk_patience:
            now = held[at] = [want, keys, 0, ctx.serial]
        else:
            now[2] += 1
            now[3] = ctx.serial
        return now[0]

    def _keys_for_the_split(self, ctx) -> int:
        if not ctx.n_single:
            return 0
        now = ctx.part_state.get(self.recording_signature, {}).get((ctx.n_single, ctx.max_seq_len))
        if now is not None and now[3] == ctx.serial:      # this step was keyed by a chunk: the figure that gives it
            return now[1]
        return ctx.single_keys(self.window)

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T = x.shape[0]
        write = self.kv_proj and cache.writes
        n_kv = self.kv_heads if self.kv_proj else 0
        qkv = ctx.workspace("attn.qkv", (T, self.q_size + 2 * n_kv * self.head_dim), self.dtype)
        rotary = self.position.rotary() if self.position is not None else None
        g = cache.group
        if self.position is None or rotary is not None:
            inv_freq, rotary_dim = (None, 0) if rotary is None else rotary[:2]
            k.qkv_rope_cache(x, self.w_qkv, qkv, ctx.positions, ctx.slot_maps[g], inv_freq, rotary_dim, cache.k, cache.v,
                             self.heads, n_kv, self.head_dim, cache.page_size, cache.num_pages, write,
                             ctx.gemm_workspace(x, self.w_qkv))
        else:     # an encoding of its own: it changes q and k between the product and the cache write
            k.gemm(x, self.w_qkv, qkv, EPI_STORE, ctx.gemm_workspace(x, self.w_qkv))
            q3 = qkv[:, :self.q_size].unflatten(1, (self.heads, self.head_dim))
            k3 = qkv[:, self.q_size:self.q_size + self.kv_size].unflatten(1, (self.kv_heads, self.head_dim)) if n_kv else None
            self.position.apply(ctx, q3, k3)
            if write:
                k.rope_kv_write(qkv, ctx.positions, ctx.slot_maps[g], None, 0, False, cache.k, cache.v,
                                self.heads, n_kv, self.head_dim, cache.page_size, cache.num_pages, write)
        o = ctx.workspace("attn.out", (T, self.q_size), self.dtype)
        # room for the partial results of single-token entries, which the kernel splits by key range
        need = k.attention_scratch_floats(ctx.n_entries, self.heads, self.head_dim, ctx.max_seq_len, self.kv_heads, ctx.n_single) if ctx.n_single else 0
        scratch = ctx.workspace("attn.partial", (need,), torch.float32) if need else None
        k.attention(qkv[:, :self.q_size], o, cache.k, cache.v, ctx.block_tables[g], ctx.token_entry, ctx.positions,
                    ctx.q_starts, ctx.seq_lens, self.heads, self.kv_heads, self.head_dim, cache.page_size,
                    cache.num_pages, self.window, self.scale, scratch, ctx.max_seq_len, ctx.n_single,
                    self._keys_for_the_split(ctx))
        leave = ctx.room_for_next_norm(h, self.w_o)
        k.gemm(o, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(o, self.w_o), **({} if leave is None else {"leave": leave}))
        ctx.note_left(h, leave)


register_mixer("attention", Attention)
