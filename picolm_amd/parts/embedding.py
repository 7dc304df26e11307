"""Token embedding and the output head.  x = table[token] widened to float, no scaling
(picolm/model_core.c:1785-1786); logits = W_out h, where W_out is the embedding table when
the checkpoint has no `lm_head.weight` (picolm/safetensors.c:248-251) or the configuration
ties them."""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import Part, Runtime


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
        if self.table is None:
            raise ValueError(f"embedding {self.name} has no table loaded")
        x = b.buffer("residual", self.D, torch.float32)
        b.embed(self.table, x)
        return x

    def forward(self, tokens: torch.Tensor, x: torch.Tensor) -> None:
        """The same on tensors, now: rows of the table for `tokens`, widened to float, into x."""
        kernels.embed(self.table, tokens, x)


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

    def emit(self, b, src) -> None:
        """logits = W h for the wanted rows h of `src`, as an operation of a launch program."""
        from ..engine.program import ROWS_WANTED
        if self.weight is None:
            raise ValueError(f"head {self.name} has no weights loaded")
        logits = b.buffer("logits", self.V, torch.float32, ROWS_WANTED)
        b.linear(self.weight, src, logits, kernels.EPI_STORE, rows=ROWS_WANTED)
        b.logits_buffer = logits

    def forward(self, h: torch.Tensor, logits: torch.Tensor) -> None:
        """The same on tensors, now."""
        kernels.gemm(h, self.weight, logits, kernels.EPI_STORE)
