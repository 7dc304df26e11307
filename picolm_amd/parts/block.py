"""Arrangements of norm, mixer and feed-forward in a layer.  PreNormBlock is picolm's
(picolm/model_core.c:1841, :2151, :2160, :2204): x += mixer(norm(x)); x += ffn(norm(x));
a block without a feed-forward skips the second half, as picolm does when the three
matrices are absent (:2159)."""
from __future__ import annotations

from .base import Block, FeedForward, Mixer, Norm


def norm_ref_of(norm):
    """The norm as the product before it may prepare it, or None for a norm of another kind."""
    f = getattr(norm, "norm_ref", None)
    return f() if f is not None else None


class PreNormBlock(Block):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, ffn: FeedForward | None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def first_norm(self):
        """The norm this block applies to the residual stream on entry: the block before may
        have it prepared."""
        return self.mixer_norm

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        """x += mixer(norm(x)); x += ffn(norm(x)) over the residual rows in buffer `x`, as operations
        of a launch program.  `after`: the RMSNorm that meets x after this block (after_when = 1: only
        in steps that want every row's logits), so that the block's last product can prepare it.
        Every part emits what it is: the engine's operations, or a call of its `forward`."""
        if type(self).forward is not Block.forward and type(self).emit is PreNormBlock.emit:
            return Block.emit(self, b, x, after, after_when)       # a subclass with an arrangement of its own
        src = self.mixer_norm.emit(b, x)
        if self.ffn is None:
            self.mixer.emit(b, src, x, after, after_when)
            return
        self.mixer.emit(b, src, x, norm_ref_of(self.ffn_norm), 0)
        self.ffn.emit(b, self.ffn_norm.emit(b, x), x, after, after_when)
