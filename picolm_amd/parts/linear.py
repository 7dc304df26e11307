"""y = x W^T for a weight W[out][in] kept as stored (picolm multiplies weights in their
file dtype with float accumulation, picolm/tensor.c:839, picolm/quant.c:4957-4968).

In the 32-bit runtime every weight is float32 (bfloat16 values widened exactly) and the
product runs on the vector ALU.  In the bfloat16 runtime a bfloat16 weight goes to the
matrix-core kernels; a weight stored in 32-bit stays 32-bit and takes the float kernel.
"""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import Part, Runtime


class Linear(Part):
    """One or several checkpoint matrices stacked along their output rows.

    `interleave=True` stacks exactly two matrices row by row (row 2j of the first, row
    2j+1 of the second): the layout the gated epilogue reads.
    """
    graph_safe = True      # launches depend on device memory only

    def __init__(self, names, out_sizes, in_size: int, interleave: bool = False):
        self.names = list(names)
        self.out_sizes = list(out_sizes)
        self.in_size = in_size
        self.interleave = interleave
        if interleave and (len(self.names) != 2 or self.out_sizes[0] != self.out_sizes[1]):
            raise ValueError("interleaving needs two matrices of equal size")
        self.weight = None

    @property
    def out_size(self) -> int:
        return sum(self.out_sizes)

    def tensor_specs(self):
        return [TensorSpec(n, (o, self.in_size)) for n, o in zip(self.names, self.out_sizes)]

    def load(self, fetch, runtime: Runtime) -> None:
        ws = [fetch.get(n) for n in self.names]
        self.set_weights(ws, runtime)

    def set_weights(self, ws, runtime: Runtime) -> None:
        if runtime.is_f32 or any(w.dtype == torch.float32 for w in ws):
            ws = [w.to(torch.float32) for w in ws]
        if self.interleave:
            w = torch.stack(ws, dim=1).reshape(self.out_size, self.in_size)
        else:
            w = ws[0] if len(ws) == 1 else torch.cat(ws, dim=0)
        self.weight = w.contiguous()

    def emit(self, b, src, out: int, epilogue: int = kernels.EPI_STORE, **kw) -> None:
        """The product as an operation of a launch program; `src` is a buffer or `Rows` (rows with
        the norm they are the result of), `kw` as ProgramBuilder.linear takes them (the rows
        covered, the norm that meets the output next)."""
        if self.weight is None:
            raise ValueError(f"product {self.names} has no weights loaded")
        b.linear(self.weight, src, out, epilogue, **kw)

    def forward(self, a: torch.Tensor, out: torch.Tensor, epilogue: int = kernels.EPI_STORE) -> None:
        """out (=, +=, = silu-gated) a W^T on tensors, now: for parts that run from Python."""
        kernels.gemm(a, self.weight, out, epilogue)
