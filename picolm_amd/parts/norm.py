"""RMSNorm: out = (x * 1/sqrt(mean(x^2) + eps)) * w, in float (picolm/tensor.c:2942-3064)."""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import Norm, Runtime, StepContext, keeps_forward


class RMSNorm(Norm):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, name: str, size: int, eps: float, weight_offset: float = 0.0):
        self.name = name
        self.size = size
        self.eps = float(eps)
        # picolm adds 1.0 to every norm weight it loads from safetensors
        # (picolm/model_core.c:954, :963), a convention of other architectures; a part of
        # such an architecture passes weight_offset=1.
        self.weight_offset = float(weight_offset)
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.size,), init="ones")]

    def load(self, fetch, runtime: Runtime) -> None:
        w = fetch.get(self.name).to(torch.float32)      # exact; picolm converts norm weights at load too (model_core.c:947-995)
        if self.weight_offset:
            w = w + self.weight_offset
        self.weight = w.contiguous()

    def norm_ref(self):
        """This norm as the products around it can carry it (they compute it on their way in and,
        in decode steps, share it between them), or None if a subclass has changed what it does."""
        from ..engine.program import NormRef
        if self.weight is None:
            raise ValueError(f"norm {self.name} has no weights loaded")
        return NormRef(self.weight, self.eps) if keeps_forward(self, RMSNorm) else None

    def emit(self, b, x: int, rows: int = 0):
        from ..engine.program import ROWS_WANTED, Rows
        ref = self.norm_ref()
        if ref is None:
            return Norm.emit(self, b, x, rows)
        return Rows(b.buffer("norm.final" if rows == ROWS_WANTED else "norm.out", self.size, b.dtype, rows), ref, x)

    def forward(self, ctx: StepContext, x, rows=None, n_rows=None, out_name="norm.out"):
        n = x.shape[0] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.ws.get(out_name, (n, self.size), ctx.dtype)
        kernels.rmsnorm(x, self.weight, self.eps, out, rows)
        return out
