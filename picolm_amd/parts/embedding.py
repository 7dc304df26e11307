"""Token embedding and the output head.  x = table[token] widened to float, no scaling
(picolm/model_core.c:1785-1786); logits = W_out h, where W_out is the embedding table when
the checkpoint has no `lm_head.weight` (picolm/safetensors.c:248-251) or the configuration
ties them."""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import NormedRows, Part, Runtime, StepContext


class TokenEmbedding(Part):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, name: str, vocab_size: int, hidden_size: int):
        self.name, self.V, self.D = name, vocab_size, hidden_size
        self.table = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.V, self.D))]

    def load(self, fetch, runtime: Runtime) -> None:
        t = fetch.get(self.name)
        self.table = (t.to(torch.float32) if runtime.is_f32 else t).contiguous()

    def emit(self, b) -> int:
        """The lookup as an operation of a launch program; returns the buffer of the residual rows."""
        from ..engine.program import CannotEmit
        if type(self) is not TokenEmbedding or self.table is None:
            raise CannotEmit(f"{type(self).__name__} is no plain embedding with a loaded table")
        x = b.buffer("residual", self.D, torch.float32)
        b.embed(self.table, x)
        return x

    def forward(self, ctx: StepContext, tokens: torch.Tensor, n_tokens: int) -> torch.Tensor:
        x = ctx.ws.get("residual", (n_tokens, self.D), torch.float32)
        kernels.embed(self.table, tokens, x)
        return x


class LMHead(Part):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, name: str, vocab_size: int, hidden_size: int, embedding: TokenEmbedding, tied: bool):
        self.name, self.V, self.D, self.embedding, self.tied = name, vocab_size, hidden_size, embedding, tied
        self.weight = None

    def tensor_specs(self):
        # optional either way: absent -> the embedding table serves; a tied model's stray
        # copy is ignored
        return [TensorSpec(self.name, (self.V, self.D), optional=True, init=None if self.tied else "normal")]

    def load(self, fetch, runtime: Runtime) -> None:
        if self.tied or not fetch.has(self.name):
            self.weight = self.embedding.table
        else:
            t = fetch.get(self.name)
            self.weight = (t.to(torch.float32) if runtime.is_f32 else t).contiguous()

    takes_normed_rows = True   # the input goes to the product unchanged

    def emit(self, b, norm, x: int) -> None:
        """logits = W norm(x) on the wanted rows, as an operation of a launch program."""
        from ..engine.program import ROWS_WANTED, CannotEmit
        if type(self) is not LMHead or self.weight is None:
            raise CannotEmit(f"{type(self).__name__} is no plain head with loaded weights")
        h = b.buffer("norm.final", self.D, b.dtype, ROWS_WANTED)
        logits = b.buffer("logits", self.V, torch.float32, ROWS_WANTED)
        b.linear(self.weight, h, logits, kernels.EPI_STORE, rows=ROWS_WANTED, in_norm=norm, in_norm_x=x)
        b.logits_buffer = logits

    def forward(self, ctx: StepContext, h) -> torch.Tensor:
        """h: the final hidden rows, or NormedRows of them."""
        logits = ctx.ws.get("logits", (h.shape[0], self.V), torch.float32)
        if isinstance(h, NormedRows):
            rms = h.norm.rms_parameters()
            hp = h.prepared[0] if h.prepared is not None else None
            if hp is not None and rms is not None and kernels.gemm_links_norms(hp, self.weight, logits, kernels.EPI_STORE, prepares=False):
                kernels.gemm_linked(hp, self.weight, logits, kernels.EPI_STORE, None, (h.prepared[1], h.x.shape[1], rms[1]))
                return logits
            h = h.tensor()
        kernels.gemm(h, self.weight, logits, kernels.EPI_STORE)
        return logits
