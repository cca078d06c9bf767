"""Arrangements of mixer, feed-forward and norms around the residual stream."""
from __future__ import annotations

from .base import Block, StepContext, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x1 = x + mixer(norm(x)); x2 = x1 + feed_forward(norm(x1)).

    src/graph/llama_like.cpp:66-105.  The residual stream stays float32; each add is
    fused into the norm that follows it, so the block returns its feed-forward
    output for the next norm (the next block's, or the model's last) to add.
    """

    def forward(self, x, pending, ctx: StepContext, line, writes_cache):
        h = self.mixer_norm.forward(x, pending, ctx)
        d = self.mixer.forward(h, ctx, line, writes_cache, self.position)
        h2 = self.feed_forward_norm.forward(x, d, ctx)
        return self.feed_forward.forward(h2, ctx)
