"""Block arrangements.  "prenorm": h += mixer(norm(h)); h += feed_forward(norm(h))
(src/arch/llama.rs:152-170).  Another arrangement (one norm for two parallel
halves, norms after the parts) is another subclass of `Block`, registered under
its own name; the parts it needs beyond these four come under the names the
layer's spec gives them in `extra`."""
from __future__ import annotations

from .base import Block, register_block


class PreNormBlock(Block):
    needs = ("mixer", "feed_forward", "mixer_norm", "feed_forward_norm")

    def forward(self, ctx, h, cache):
        x = ctx.workspace("block.x", (h.shape[0], h.shape[1]), self.mixer.dtype)
        self.mixer_norm.forward(ctx, h, x)
        self.mixer.forward(ctx, x, h, cache)
        self.feed_forward_norm.forward(ctx, h, x)
        self.feed_forward.forward(ctx, x, h)


register_block("prenorm", PreNormBlock)
