"""Arrangements of norm, mixer and feed-forward in a layer.  PreNormBlock is picolm's
(picolm/model_core.c:1841, :2151, :2160, :2204): x += mixer(norm(x)); x += ffn(norm(x));
a block without a feed-forward skips the second half, as picolm does when the three
matrices are absent (:2159)."""
from __future__ import annotations

from .base import Block, FeedForward, Mixer, Norm, StepContext


class PreNormBlock(Block):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, ffn: FeedForward | None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def first_norm(self):
        """The norm this block applies to the residual stream on entry: the block before may
        have it prepared (see NormedRows)."""
        return self.mixer_norm

    def forward(self, ctx: StepContext, x) -> None:
        """x += mixer(norm(x)); x += ffn(norm(x))."""
        after = ctx.norm_after_block                # the norm that meets x after this block, if the caller knows it
        h = ctx.normed(self.mixer_norm, x, self.mixer)
        ctx.norm_after = self.ffn_norm if self.ffn is not None else after
        self.mixer.forward(ctx, h, x)
        if self.ffn is not None:
            h = ctx.normed(self.ffn_norm, x, self.ffn)
            ctx.norm_after = after
            self.ffn.forward(ctx, h, x)
        ctx.norm_after = None
