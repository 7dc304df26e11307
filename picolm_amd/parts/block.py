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

    def forward(self, ctx: StepContext, x) -> None:
        h = self.mixer_norm.forward(ctx, x)
        self.mixer.forward(ctx, h, x)
        if self.ffn is not None:
            h = self.ffn_norm.forward(ctx, x)
            self.ffn.forward(ctx, h, x)
