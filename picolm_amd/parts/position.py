"""Position encodings.  Rotary: tables cos/sin[pos][i] of pos * f_i with f_i = theta^(-2i/d)
(picolm/model_core.c:314-326), optionally with the "llama3" wavelength-dependent scaling of
the frequencies, which picolm does not have; the rotation itself runs fused with the cache
write.  Frequencies are computed in float64 and rounded once; the angle pos * f_i and its
cosine and sine are 32-bit, as picolm's are."""
from __future__ import annotations

import math

import torch

from .base import PositionEncoding, Runtime

STYLES = {"pairwise": 0, "half": 1}


def rotary_inv_freq(head_dim: int, theta: float, scaling=None) -> torch.Tensor:
    i = torch.arange(head_dim // 2, dtype=torch.float64)
    inv = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * i / head_dim)
    if scaling is None:
        return inv
    factor, low, high = scaling.factor, scaling.low_freq_factor, scaling.high_freq_factor
    orig = float(scaling.original_max_position_embeddings)
    wavelen = 2.0 * math.pi / inv
    smooth = (orig / wavelen - low) / (high - low)
    blended = (1.0 - smooth) * inv / factor + smooth * inv
    out = torch.where(wavelen > orig / low, inv / factor, blended)
    return torch.where(wavelen < orig / high, inv, out)


class RotaryEmbedding(PositionEncoding):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, head_dim: int, theta: float, scaling=None, style: str = "pairwise"):
        if head_dim % 2:
            raise ValueError(f"rotary head size {head_dim} is odd")
        if style not in STYLES:
            raise ValueError(f"rotary pairing '{style}' is not one of {sorted(STYLES)}")
        self.head_dim, self.theta, self.scaling, self.style = head_dim, float(theta), scaling, style
        self.cos = self.sin = None
        self.n_positions = 0
        self._handed_out = []       # earlier, shorter tables: recorded steps hold their addresses

    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        if self.cos is not None and self.n_positions >= max_positions and self.cos.device == runtime.device:
            return
        if self.cos is not None:
            # a recorded decode step keeps the raw addresses of the tables it was recorded with and
            # no reference to them: tables that were handed out are kept for the part's lifetime
            self._handed_out.append((self.cos, self.sin))
        inv = rotary_inv_freq(self.head_dim, self.theta, self.scaling).to(torch.float32)
        pos = torch.arange(max_positions, dtype=torch.float32)
        ang = pos[:, None] * inv[None, :]                     # float32 product
        # cos/sin of the 32-bit angle, evaluated in float64 and rounded: correctly rounded
        # values, independent of the device's libm
        self.cos = torch.cos(ang.double()).float().contiguous().to(runtime.device)
        self.sin = torch.sin(ang.double()).float().contiguous().to(runtime.device)
        self.n_positions = max_positions

    def rotary_tables(self):
        return self.cos, self.sin, STYLES[self.style]


class NoPosition(PositionEncoding):
    """Keys and queries are used as projected."""
    graph_safe = True      # launches depend on device memory only

