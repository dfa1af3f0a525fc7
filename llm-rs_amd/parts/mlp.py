"""SwiGLU feed-forward(hidden_size, intermediate_size):
h += (silu(x Wg^T) * (x Wu^T)) Wd^T, silu(v) = v / (1 + exp(-v))
(src/arch/llama.rs:165-170, shaders/ops.metal:762-793).  The gate and up weights
are interleaved row by row at load, so one product yields (gate_j, up_j) side by
side and its epilogue writes silu(gate) * up, computed in 32-bit, once; the down
product adds into the 32-bit residual stream.  No biases."""
from __future__ import annotations

import torch

from ..kernels import EPI_ACCUM_F32, EPI_SWIGLU, kernels
from .base import FeedForward, TensorSpec, place, register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.w_gate_up = None
        self.w_down = None

    def tensors(self):
        return {self.name("gate_proj.weight"): TensorSpec((self.inter, self.hidden)),
                self.name("up_proj.weight"): TensorSpec((self.inter, self.hidden)),
                self.name("down_proj.weight"): TensorSpec((self.hidden, self.inter))}

    def load(self, tensors, device):
        gate = place(tensors[self.name("gate_proj.weight")], device, self.dtype)
        up = place(tensors[self.name("up_proj.weight")], device, self.dtype)
        self.w_gate_up = torch.stack([gate, up], dim=1).reshape(2 * self.inter, self.hidden).contiguous()
        self.w_down = place(tensors[self.name("down_proj.weight")], device, self.dtype)

    def export(self):
        both = self.w_gate_up.cpu().view(self.inter, 2, self.hidden)
        return {self.name("gate_proj.weight"): both[:, 0, :].contiguous(), self.name("up_proj.weight"): both[:, 1, :].contiguous(),
                self.name("down_proj.weight"): self.w_down.cpu()}

    def takes_normed_rows(self, ctx, rows):
        return kernels().product_norms_its_rows(rows, 2 * self.inter, self.hidden, self.dtype)

    def forward(self, ctx, x, h):
        k = kernels()
        act = ctx.workspace("mlp.act", (x.shape[0], self.inter), self.dtype)
        k.gemm(x, self.w_gate_up, act, EPI_SWIGLU, ctx.gemm_workspace(x, self.w_gate_up))
        leave = ctx.room_for_next_norm(h, self.w_down)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down), **({} if leave is None else {"leave": leave}))
        ctx.note_left(h, leave)


register_feed_forward("swiglu", SwiGLU)
