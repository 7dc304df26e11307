"""Sampling options with picolm's names and meanings (picolm/sampler.h:6-12, sampler.c:37-44).

The library's defaults switch every filter off (greedy, no top-k, top_p 1, min_p 0); the
command line uses picolm's defaults (picolm/picolm.c:774-777, :1230).
"""
from __future__ import annotations

from dataclasses import dataclass

MASK64 = (1 << 64) - 1
_STREAM_STEP = 0x9E3779B97F4A7C15


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0      # <= 0: greedy, the first maximum
    top_k: int = 0                # 0 or >= vocabulary: off
    top_p: float = 1.0            # cumulative probability kept, measured before the temperature
    min_p: float = 0.0            # drop tokens below min_p * the largest probability
    seed: int = 42                # 0 becomes 42

    def validate(self) -> None:
        if self.top_k < 0:
            raise ValueError(f"top_k: {self.top_k} is negative")
        if not self.top_p > 0.0:
            raise ValueError(f"top_p: {self.top_p} must be positive")
        if self.min_p < 0.0:
            raise ValueError(f"min_p: {self.min_p} is negative")

    @property
    def greedy(self) -> bool:
        return not self.temperature > 0.0


CLI_DEFAULTS = SamplingParams(temperature=0.8, top_k=40, top_p=0.9, min_p=0.05, seed=42)


def stream_state(seed: int, index: int) -> int:
    """Initial xorshift64 state of sequence `index`: sequence 0 has picolm's single stream
    (`seed ? seed : 42`, picolm/sampler.c:43); the others are offset so that a sequence's
    draws do not depend on what else is in its batch."""
    s = (int(seed) & MASK64) or 42
    s = (s + index * _STREAM_STEP) & MASK64
    return s or 42
