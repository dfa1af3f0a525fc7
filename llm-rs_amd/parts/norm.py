"""RMSNorm(size, eps): y = x / sqrt(mean(x^2) + eps) * weight, computed in 32-bit,
the weight multiplying directly.  Reference: rms_norm_batch
(shaders/ops.metal:970-1003), used at src/arch/llama.rs:152,164,135."""
from __future__ import annotations

import torch

from ..kernels import NormedRows, kernels
from .base import Norm, TensorSpec, place, register_norm


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight = None

    def tensors(self):
        return {self.name("weight"): TensorSpec((self.size,), "norm")}

    def load(self, tensors, device):
        # The reference wants norm weights in 32-bit (ops.metal:972); whatever the
        # file stores, the kernel multiplies by a float32 weight.
        self.weight = place(tensors[self.name("weight")], device, torch.float32)

    def export(self):
        return {self.name("weight"): self.weight.cpu()}

    def forward(self, ctx, h, out, rows=None):
        kernels().rmsnorm(out, h, self.weight, self.eps, rows)

    def deferred_weight(self):
        return self.weight

    def deferred_eps(self):
        return self.eps

    def deferred(self, ctx, h):
        left = ctx.left_for(h)
        if left is None or left.weight is not self.weight or h.shape[1] != self.size or left.y.shape != h.shape:
            return None         # nothing was left, or it was prepared for another norm
        if left.whole:          # finished by the product that added into the stream last
            return left.y if left.eps == self.eps else None
        return NormedRows(left.y, left.sumsq, self.eps)


register_norm("rmsnorm", RMSNorm)
