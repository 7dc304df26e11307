"""RMSNorm: out = (x * 1/sqrt(mean(x^2) + eps)) * w, in float (picolm/tensor.c:2942-3064)."""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import Norm, Runtime, StepContext


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

    def rms_parameters(self):
        return self.weight, self.eps

    def norm_ref(self):
        """This norm as a launch program's operations carry it."""
        from ..engine.program import CannotEmit, NormRef
        if type(self) is not RMSNorm or self.weight is None:
            raise CannotEmit(f"{type(self).__name__} is no plain RMSNorm with loaded weights")
        return NormRef(self.weight, self.eps)

    def forward(self, ctx: StepContext, x, rows=None, n_rows=None, out_name="norm.out"):
        n = x.shape[0] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.ws.get(out_name, (n, self.size), ctx.dtype)
        kernels.rmsnorm(x, self.weight, self.eps, out, rows)
        return out
