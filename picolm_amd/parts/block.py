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

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        """The block as operations of a launch program over the residual rows in buffer `x`;
        `after`: the norm that meets x after this block (after_when = 1: only in steps that want
        every row's logits), so that the block's last product can prepare it."""
        from ..engine.program import CannotEmit
        if type(self) is not PreNormBlock:
            raise CannotEmit(f"{type(self).__name__} changes what PreNormBlock does")
        for part in (self.mixer, self.ffn):
            if part is not None and not callable(getattr(part, "emit", None)):
                raise CannotEmit(f"{type(part).__name__} has no operations of the engine's")
        n1 = self.mixer_norm.norm_ref() if hasattr(self.mixer_norm, "norm_ref") else None
        if n1 is None:
            raise CannotEmit(f"{type(self.mixer_norm).__name__} has no operations of the engine's")
        if self.ffn is None:
            self.mixer.emit(b, n1, x, after, after_when)
            return
        if not hasattr(self.ffn_norm, "norm_ref"):
            raise CannotEmit(f"{type(self.ffn_norm).__name__} has no operations of the engine's")
        n2 = self.ffn_norm.norm_ref()
        self.mixer.emit(b, n1, x, n2, 0)
        self.ffn.emit(b, n2, x, after, after_when)

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
