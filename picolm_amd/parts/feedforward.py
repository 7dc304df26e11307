"""Gated feed-forward: down(silu(gate x) * (up x)), no bias (picolm/model_core.c:2182-2204,
silu picolm/tensor.c:3306-3315).  gate and up are one product over row-interleaved weights
whose epilogue applies silu(g) * u; the down product adds into the residual."""
from __future__ import annotations

from .. import kernels
from .base import FeedForward, StepContext, keeps_forward
from .linear import Linear


class SwiGLU(FeedForward):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight")):
        self.D, self.F = hidden_size, intermediate_size
        self.gate_up = Linear([prefix + names[0], prefix + names[1]], [intermediate_size] * 2, hidden_size,
                              interleave=True)
        self.down = Linear([prefix + names[2]], [hidden_size], intermediate_size)

    def children(self):
        return [self.gate_up, self.down]

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += down(silu(gate h) * (up h)) for the rows h of `src`, as operations of a launch program."""
        if not keeps_forward(self, SwiGLU):
            return FeedForward.emit(self, b, src, x, out_norm, out_norm_when)
        act = b.buffer("ffn.act", self.F, b.dtype)
        self.gate_up.emit(b, src, act, kernels.EPI_SWIGLU)
        self.down.emit(b, act, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)

    def forward(self, ctx: StepContext, h, residual) -> None:
        """The same on tensors, now: for parts that run from Python (a routed feed-forward calls
        its experts on the rows it sends them)."""
        act = ctx.ws.get("ffn.act", (h.shape[0], self.F), ctx.dtype)
        self.gate_up.forward(h, act, kernels.EPI_SWIGLU)
        self.down.forward(act, residual, kernels.EPI_ACCUMULATE)
