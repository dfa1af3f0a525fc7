"""Block arrangements.  "prenorm": h += mixer(norm(h)); h += feed_forward(norm(h))
(src/arch/llama.rs:152-170).  "mixer_only" has no feed-forward."""
from __future__ import annotations

from .base import Block, register_block


class PreNormBlock(Block):
    def forward(self, ctx, h, cache):
        x = ctx.workspace("block.x", (h.shape[0], h.shape[1]), self.mixer.dtype)
        self.mixer_norm.forward(ctx, h, x)
        self.mixer.forward(ctx, x, h, cache)
        self.feed_forward_norm.forward(ctx, h, x)
        self.feed_forward.forward(ctx, x, h)


register_block("prenorm", PreNormBlock)
