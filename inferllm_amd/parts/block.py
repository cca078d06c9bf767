"""Arrangements of mixer, feed-forward and norms around the residual stream."""
from __future__ import annotations

from ..kernels import ops
from .base import Block, StepContext, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x1 = x + mixer(norm(x)); x2 = x1 + feed_forward(norm(x1)).

    src/graph/llama_like.cpp:66-105.  The residual stream stays float32; each add is
    fused into the norm that follows it, so the block returns its feed-forward
    output for the next norm (the next block's, or the model's last) to add.  For steps of
    few rows, parts that say so (`Part.adds_residual`, `takes_normed_rows`) shorten this: a
    part adds its output to the stream in its last kernel, which also prepares the norm that
    follows for the next part's first kernel; what the block hands on is then None (nothing
    left to add) or `ops.NormedRows`.
    """

    graph_safe_prompts = True

    takes_next_norm = True
    takes_prepared_rows = True

    @staticmethod
    def _enter(norm, part, x, pending, ctx):
        """The input of `part`: the normed rows of x (+ pending), by a kernel or prepared."""
        if isinstance(pending, ops.NormedRows):
            params = norm.rms_params()
            if params is not None and pending.made_for(*params):
                return pending if part.takes_normed_rows else pending.rows()
            pending = None                       # the sum is in x already; another norm follows
        return norm.forward(x, pending, ctx)

    def forward(self, x, pending, ctx: StepContext, line, writes_cache, next_norm=None):
        h = self._enter(self.mixer_norm, self.mixer, x, pending, ctx)
        if self.mixer.adds_residual:
            d = self.mixer.forward(h, ctx, line, writes_cache, self.position, residual=x,
                                   next_norm=self.feed_forward_norm)
        else:
            d = self.mixer.forward(h, ctx, line, writes_cache, self.position)
        h2 = self._enter(self.feed_forward_norm, self.feed_forward, x, d, ctx)
        if self.feed_forward.adds_residual:
            return self.feed_forward.forward(h2, ctx, residual=x, next_norm=next_norm)
        return self.feed_forward.forward(h2, ctx)
