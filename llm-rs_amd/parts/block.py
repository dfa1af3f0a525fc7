"""Block arrangements.  "prenorm": h += mixer(norm(h)); h += feed_forward(norm(h))
(src/arch/llama.rs:152-170).  Another arrangement (one norm for two parallel
halves, norms after the parts) is another subclass of `Block`, registered under
its own name; the parts it needs beyond these four come under the names the
layer's spec gives them in `extra`."""
from __future__ import annotations

from .base import Block, register_block


class PreNormBlock(Block):
    needs = ("mixer", "feed_forward", "mixer_norm", "feed_forward_norm")
    keeps_left_current = True       # `normed_input` drops what was left before each part; the feed-forward runs last

    def first_norm(self):
        return self.mixer_norm

    def forward(self, ctx, h, cache):
        after = ctx.norm_after_block
        self.mixer.forward(ctx, self.normed_input(ctx, h, self.mixer_norm, self.mixer, self.feed_forward_norm), h, cache)
        self.feed_forward.forward(ctx, self.normed_input(ctx, h, self.feed_forward_norm, self.feed_forward, after), h)
        ctx.upcoming_norm = None


register_block("prenorm", PreNormBlock)
