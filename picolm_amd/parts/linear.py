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
from .base import NormedRows, Part, Runtime


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

    def emit(self, b, inp: int, out: int, epilogue: int = kernels.EPI_STORE, **norms) -> None:
        """The same product as an operation of a launch program; `norms` as ProgramBuilder.linear
        takes them (the norm of the input, the norm that meets the output next)."""
        from ..engine.program import CannotEmit
        if type(self) is not Linear or self.weight is None:
            raise CannotEmit(f"{type(self).__name__} is no plain Linear with loaded weights")
        b.linear(self.weight, inp, out, epilogue, **norms)

    def forward(self, a, out: torch.Tensor, epilogue: int = kernels.EPI_STORE, ctx=None) -> None:
        """out (=, +=, = silu-gated) a W^T.  `a` is a tensor, or NormedRows: rows whose norm the
        products compute between them.  With `ctx` and the accumulating epilogue, the norm that
        the context says comes after (`ctx.norm_after`) is prepared for the product that follows,
        where the kernels can do that; the result is left in `ctx.prepared_norm`."""
        prepared = None
        if isinstance(a, NormedRows):
            rms = a.norm.rms_parameters()
            h = a.prepared[0] if a.prepared is not None else None
            if h is not None and rms is not None and kernels.gemm_links_norms(h, self.weight, out, epilogue, prepares=False):
                prepared = (a.prepared[1], a.x.shape[1], rms[1])
                a = h
            else:
                a = a.tensor()
        prepare = None
        nxt = ctx.norm_after if ctx is not None and epilogue == kernels.EPI_ACCUMULATE else None
        if nxt is not None and nxt.rms_parameters() is not None and kernels.gemm_links_norms(a, self.weight, out, epilogue, prepares=True):
            T, N = out.shape
            which = ctx.ws.flip("norm.prepared")
            prepare = (nxt.rms_parameters()[0], ctx.ws.get(f"norm.prepared.h{which}", (T, N), torch.bfloat16),
                       ctx.ws.get(f"norm.prepared.ssq{which}", (kernels.linked_norm_parts(T, N, a.shape[1]), kernels.linked_norm_rows(T)),
                                  torch.float32))
        if prepare is None and prepared is None:
            kernels.gemm(a, self.weight, out, epilogue)
            return
        kernels.gemm_linked(a, self.weight, out, epilogue, prepare, prepared)
        if prepare is not None:
            ctx.prepared_norm = NormedRows(ctx, nxt, out, prepared=(prepare[1], prepare[2]))
