"""The sampler the engine uses: one GPU kernel call per step over the rows of logits."""
from __future__ import annotations

import torch

from .. import kernels
from .params import SamplingParams, stream_state


def _as_i64(u: int) -> int:
    return u - (1 << 64) if u >= (1 << 63) else u


class Sampler:
    """Holds one generator state per sequence on the device."""

    def __init__(self, params: SamplingParams, n_sequences: int, device):
        params.validate()
        self.params = params
        self.device = torch.device(device)
        self.n = n_sequences
        states = [_as_i64(stream_state(params.seed, i)) for i in range(n_sequences)]
        self.states = torch.tensor(states, dtype=torch.int64).to(self.device)
        self._out = torch.zeros(max(n_sequences, 1), dtype=torch.int32, device=self.device)
        # the tokens come back through pinned memory: one copy, no staging buffer; two blocks in
        # turn, so that one draw's tokens can still be on their way while the next is launched
        self._host_out = [torch.zeros(max(n_sequences, 1), dtype=torch.int32) for _ in range(2)]
        if self.device.type == "cuda":
            self._host_out = [h.pin_memory() for h in self._host_out]
        self._arrived = [torch.cuda.Event() for _ in range(2)] if self.device.type == "cuda" else [None, None]
        self._turn = 0
        self._scratch = None
        self._sample_scratch = None
        self._idx_of = None                   # the sequence indices that `_idx` holds
        self._idx = None

    def sample(self, logits: torch.Tensor, sequence_indices) -> list[int]:
        """`logits[i]` belongs to sequence `sequence_indices[i]`; returns one token each."""
        return self.launch(logits, sequence_indices).wait()

    def launch(self, logits: torch.Tensor, sequence_indices) -> "PendingTokens":
        """Start the draw and the tokens' way to the host without waiting for either.  The
        result's device tensor is the sampler's own and is written again by the next launch (in
        stream order, so work handed to the stream before that still reads these tokens); at
        most two results may be waited for at a time."""
        n = logits.shape[0]
        out = self._out[:n]
        p = self.params
        if p.greedy:
            need = kernels.argmax_scratch_floats(n, logits.shape[1])
            if self._scratch is None or self._scratch.numel() < need:
                self._scratch = torch.empty(need, dtype=torch.float32, device=self.device)
            kernels.argmax(logits, out, self._scratch)
        else:
            seqs = list(sequence_indices)
            if seqs != self._idx_of:          # the same batch step after step: one upload
                self._idx = torch.tensor(seqs, dtype=torch.int32).to(self.device)
                self._idx_of = seqs
            need = kernels.sample_scratch_bytes(n, logits.shape[1], p.temperature, p.top_k)
            if need and (self._sample_scratch is None or self._sample_scratch.numel() < need):
                self._sample_scratch = torch.empty(need, dtype=torch.uint8, device=self.device)
            kernels.sample(logits, out, p.temperature, p.top_k, p.top_p, p.min_p, self.states, self._idx,
                           self._sample_scratch if need else None)
        t = self._turn
        self._turn ^= 1
        host = self._host_out[t][:n]
        host.copy_(out, non_blocking=True)
        if self._arrived[t] is not None:
            self._arrived[t].record()
        return PendingTokens(out, host, self._arrived[t])


class PendingTokens:
    """Tokens that a sampling kernel has drawn or will have drawn: on the device for a step that
    follows at once, on the host after `wait`."""

    def __init__(self, device_tokens: torch.Tensor, host_tokens: torch.Tensor, arrived):
        self._device, self._host, self._arrived = device_tokens, host_tokens, arrived

    def on_device(self, rows=None) -> torch.Tensor:
        """The tokens as an int32 tensor on the device; `rows` picks some of them, in that order."""
        if rows is None:
            return self._device
        # the picked rows' indices go up through pinned memory without waiting for the GPU (torch
        # keeps the pinned block until the copy has run); the gather is queued behind the draw
        idx = torch.tensor(list(rows), dtype=torch.int64)
        if self._device.is_cuda:
            idx = idx.pin_memory().to(self._device.device, non_blocking=True)
        return self._device.index_select(0, idx)

    def wait(self) -> list[int]:
        if self._arrived is not None:
            self._arrived.synchronize()
        return self._host.tolist()
