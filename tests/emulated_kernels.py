"""A stand-in for the device kernels, for tests of the engine's host logic on a
machine without a GPU: the same methods as `llm_rs_amd.kernels.HipKernels`, on CPU
tensors, with the cache layouts and the rounding points of the real kernels.  It
is test equipment: the package never loads it, and the `gpu` tests do not use it.
"""
from __future__ import annotations

import math

import torch

from llm_rs_amd.kernels import Kernels, NormPlan

EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU = 0, 1, 2, 3


class EmulatedKernels(Kernels):
    """(What `Kernels` answers by itself stays: no workspace, no scratch, nothing split.)"""

    def embed_rows(self, out, table, tokens, scale=1.0):
        out.copy_(table[tokens.long()].float() * scale)

    def scale_softcap_rows(self, logits, scale, cap):
        logits.mul_(scale)
        if cap > 0:
            logits.copy_(cap * torch.tanh(logits / cap))

    def cast(self, dst, src):
        dst.copy_(src.to(dst.dtype))

    def rmsnorm(self, out, x, weight, eps, rows=None):
        src = x if rows is None else x[rows.long()]
        ss = (src * src).sum(-1, keepdim=True)
        inv = 1.0 / torch.sqrt(ss / src.shape[-1] + eps)
        out.copy_((src * inv * weight).to(out.dtype))

    # as the device: steps of up to 16 tokens in bfloat16 leave their norms to the products around them
    def product_norms_its_rows(self, M, N, K, dtype):
        return dtype == torch.bfloat16 and 1 <= M <= 16

    def norm_left_by_product(self, M, N, K, dtype):
        return NormPlan(False, -(-N // 16)) if dtype == torch.bfloat16 and 1 <= M <= 16 else None

    def gemm(self, a, w, out, epilogue=EPI_STORE, workspace=None, leave=None):
        inv = None
        if hasattr(a, "sumsq"):        # kernels.NormedRows: rows times the norm's weight, rounded; the scale comes after the sums
            inv = 1.0 / torch.sqrt(a.sumsq.sum(-1, keepdim=True) / a.y.shape[1] + a.eps)
            a = a.y
        acc = a.float() @ w.float().T
        if inv is not None:
            acc = acc * inv
        if leave is not None:          # kernels.NextNorm, with the += epilogue
            new = out + acc
            pad = torch.zeros((new.shape[0], leave.sumsq.shape[1] * 16))
            pad[:, :new.shape[1]] = new
            leave.sumsq.copy_((pad * pad).view(new.shape[0], -1, 16).sum(-1))
            leave.y.copy_((new * leave.weight).to(leave.y.dtype))
        if epilogue == EPI_STORE:
            out.copy_(acc.to(out.dtype))
        elif epilogue == EPI_STORE_F32:
            out.copy_(acc)
        elif epilogue == EPI_ACCUM_F32:
            out.add_(acc)
        else:
            g, u = acc[:, 0::2], acc[:, 1::2]
            out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))

    def rope_kv_write(self, qkv, positions, slot_map, inv_freq, rotary_dim, interleaved, k_cache, v_cache,
                      n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv):
        T = qkv.shape[0]
        heads = qkv[:, :(n_heads + 2 * n_kv_heads) * head_dim].view(T, n_heads + 2 * n_kv_heads, head_dim)
        n_rot = n_heads + n_kv_heads
        x = heads[:, :n_rot, :].float()
        if rotary_dim:
            angle = positions.float()[:, None] * inv_freq[None, :]
            cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
            y = x.clone()
            r = rotary_dim
            if interleaved:
                a, b = x[..., 0:r:2], x[..., 1:r:2]
                y[..., 0:r:2], y[..., 1:r:2] = a * cos - b * sin, a * sin + b * cos
            else:
                a, b = x[..., :r // 2], x[..., r // 2:r]
                y[..., :r // 2], y[..., r // 2:r] = a * cos - b * sin, a * sin + b * cos
            x = y
        x = x.to(qkv.dtype)
        heads[:, :n_heads, :] = x[:, :n_heads, :]
        if not write_kv:
            return
        kc = k_cache.view(num_pages, n_kv_heads, page_size, head_dim)
        vc = v_cache.view(num_pages, n_kv_heads, head_dim, page_size)
        page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
        for t in range(T):
            kc[page[t], :, off[t], :] = x[t, n_heads:, :]
            vc[page[t], :, :, off[t]] = heads[t, n_rot:, :]

    def qkv_rope_cache(self, x, w, qkv, positions, slot_map, inv_freq, rotary_dim, k_cache, v_cache,
                       n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv, workspace=None):
        if hasattr(x, "sumsq"):        # the device rotates the 32-bit sums and rounds once; so does this
            full = torch.empty(qkv.shape, dtype=torch.float32)
            self.gemm(x, w, full, EPI_STORE_F32)
            self.rope_kv_write(full, positions, slot_map, inv_freq, rotary_dim, True, k_cache, v_cache,
                               n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv)
            qkv.copy_(full.to(qkv.dtype))
            return
        self.gemm(x, w, qkv, EPI_STORE)
        self.rope_kv_write(qkv, positions, slot_map, inv_freq, rotary_dim, True, k_cache, v_cache,
                           n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv)

    def attention(self, q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, seq_lens,
                  n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale, scratch=None, max_seq_len=0, n_single=-1,
                  single_keys=0):
        T = q.shape[0]
        kc = k_cache.view(num_pages, n_kv_heads, page_size, head_dim).float()
        vc = v_cache.view(num_pages, n_kv_heads, head_dim, page_size).float()
        rep = n_heads // n_kv_heads
        for t in range(T):
            pos = int(positions[t])
            table = block_table[int(token_entry[t])]
            lo = max(0, pos + 1 - window) if window > 0 else 0
            js = torch.arange(lo, pos + 1)
            pages, offs = table[js // page_size].long(), js % page_size
            keys = kc[pages, :, offs, :]                       # [n, kv, d]
            vals = vc[pages, :, :, offs]                       # [n, kv, d]
            qt = q[t, :n_heads * head_dim].view(n_heads, head_dim).float()
            for h in range(n_heads):
                g = h // rep
                s = (keys[:, g, :] @ qt[h]) * scale
                p = torch.softmax(s, dim=0)
                out[t, h * head_dim:(h + 1) * head_dim] = (p @ vals[:, g, :]).to(out.dtype)

    def argmax_rows(self, logits, out, scratch=None):
        for i in range(logits.shape[0]):
            best = logits[i].max()
            out[i] = int((logits[i] == best).nonzero()[0])

    def place_ids(self, tokens, rows, sources, ids, vocab):
        for row, src in zip(rows.tolist(), sources.tolist()):
            if 0 <= row < tokens.numel() and 0 <= src < ids.numel() and 0 <= int(ids[src]) < vocab:
                tokens[row] = ids[src]

    def sample_rows(self, logits, words, out):
        w = words.cpu()
        for i in range(logits.shape[0]):
            u = w[i, 0:1].view(torch.float32).item()
            temp = w[i, 1:2].view(torch.float32).item()
            top_k = int(w[i, 2])
            top_p = w[i, 3:4].view(torch.float32).item()
            row = logits[i]
            V = row.shape[0]
            if temp == 0.0:
                out[i] = int((row == row.max()).nonzero()[0])
                continue
            z = row * (1.0 / temp)
            order = sorted(range(V), key=lambda j: (-float(z[j]), j))
            keep = torch.ones(V, dtype=torch.bool)
            if 0 < top_k < V:
                keep[:] = False
                keep[order[:top_k]] = True
            p = torch.softmax(z.masked_fill(~keep, float("-inf")), dim=0)
            if top_p < 1.0:
                total, cut = 0.0, V
                for n, j in enumerate(order):
                    total += float(p[j])
                    if total >= top_p:
                        cut = n + 1
                        break
                p[order[cut:]] = 0.0
                p = p / p.sum()
            hit = (torch.cumsum(p, 0) > u).nonzero()
            out[i] = int(hit[0]) if len(hit) else int(p.nonzero()[-1])
