"""Random-weights mode: the tensors a model declares, filled from a seed.

picolm has nothing like it (nearest: `srand48(42)` blocks in its kernel diff,
picolm/picolm.c:577-593).  Each tensor has a stream of its own, derived from the seed and
the tensor's name, so a tensor's values do not depend on which others are made.  Matrices
are N(0, std); norm weights are 1, or 1 + N(0, norm_sigma).
"""
from __future__ import annotations

import json
import os
import zlib

import torch

from .checkpoint import TensorDict, TensorSpec
from .safetensors_io import write_safetensors

_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _stream_seed(seed: int, name: str) -> int:
    return (int(seed) * 0x9E3779B1 + zlib.crc32(name.encode("utf-8"))) & 0x7FFFFFFFFFFFFFFF


def random_tensor(spec: TensorSpec, seed: int, std: float, norm_sigma: float,
                  dtype: torch.dtype, device="cpu") -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(_stream_seed(seed, spec.name))
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "ones":
        t = torch.ones(spec.shape, dtype=torch.float32, device=device)
        if norm_sigma > 0:
            t += torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device) * norm_sigma
    else:
        t = torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device) * std
    return t.to(dtype)


def random_tensors(specs, seed: int, std: float = 0.02, norm_sigma: float = 0.0,
                   dtype: torch.dtype = torch.bfloat16, device="cpu"):
    """Yield (name, tensor) for every spec that random mode writes."""
    for s in specs:
        if s.init is None:
            continue
        yield s.name, random_tensor(s, seed, std, norm_sigma, dtype, device)


class RandomWeights(TensorDict):
    """A weight source that makes each tensor when it is asked for, on `device`; nothing is
    kept, so a model of any size can be filled without a file."""

    def __init__(self, specs, seed, std=0.02, norm_sigma=0.0, dtype=torch.bfloat16, device="cpu"):
        self.source = f"<random seed={seed}>"
        self._specs = {s.name: s for s in specs if s.init is not None}
        self._args = (seed, std, norm_sigma, dtype, device)

    def names(self):
        return list(self._specs)

    def info(self, name):
        return self._args[3], tuple(self._specs[name].shape)

    def tensor(self, name):
        seed, std, sigma, dtype, device = self._args
        return random_tensor(self._specs[name], seed, std, sigma, dtype, device)


def write_random_model(config, out_dir: str, seed: int, std: float = 0.02, norm_sigma: float = 0.0,
                       dtype: str | None = None) -> str:
    """Write `config.json` and `model.safetensors` for `config` into `out_dir`."""
    from ..engine.builder import tensor_specs_for          # late: engine imports weights
    dtype_name = dtype or config.torch_dtype
    specs = tensor_specs_for(config)
    os.makedirs(out_dir, exist_ok=True)
    cfg = config.to_dict()
    cfg["torch_dtype"] = dtype_name
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(
        os.path.join(out_dir, "model.safetensors"),
        lambda: random_tensors(specs, seed, std, norm_sigma, _DTYPE[dtype_name]),
        metadata={"format": "pt", "seed": seed, "std": std, "norm_sigma": norm_sigma})
    return out_dir
