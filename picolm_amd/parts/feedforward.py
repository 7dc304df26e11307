"""Gated feed-forward: down(silu(gate x) * (up x)), no bias (picolm/model_core.c:2182-2204,
silu picolm/tensor.c:3306-3315).  gate and up are one product over row-interleaved weights
whose epilogue applies silu(g) * u; the down product adds into the residual."""
from __future__ import annotations

from .. import kernels
from .base import FeedForward, StepContext
from .linear import Linear


class SwiGLU(FeedForward):
    graph_safe = True      # launches depend on device memory only
    takes_normed_rows = True   # the input goes to a Linear unchanged

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight")):
        self.D, self.F = hidden_size, intermediate_size
        self.gate_up = Linear([prefix + names[0], prefix + names[1]], [intermediate_size] * 2, hidden_size,
                              interleave=True)
        self.down = Linear([prefix + names[2]], [hidden_size], intermediate_size)

    def children(self):
        return [self.gate_up, self.down]

    def emit(self, b, norm, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += down(silu(gate h) * (up h)) with h = norm(x), as operations of a launch program."""
        import torch
        from ..engine.program import CannotEmit
        if type(self) is not SwiGLU:
            raise CannotEmit(f"{type(self).__name__} changes what SwiGLU does")
        h = b.buffer("norm.out", self.D, b.dtype)
        act = b.buffer("ffn.act", self.F, b.dtype)
        self.gate_up.emit(b, h, act, kernels.EPI_SWIGLU, in_norm=norm, in_norm_x=x)
        self.down.emit(b, act, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)

    def forward(self, ctx: StepContext, h, residual) -> None:
        act = ctx.ws.get("ffn.act", (h.shape[0], self.F), ctx.dtype)
        self.gate_up.forward(h, act, kernels.EPI_SWIGLU)
        self.down.forward(act, residual, kernels.EPI_ACCUMULATE, ctx)
