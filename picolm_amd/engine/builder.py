"""From a model folder (or a configuration and random weights) to a model on the GPU."""
from __future__ import annotations

import torch

from ..config import read_config_json, resolve
from ..parts.base import Runtime
from ..weights import Checkpoint, RandomWeights
from . import llama as _llama  # noqa: F401  (registers the architecture)

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32,
           "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype {name}: the engine runs in bfloat16 or float32")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype '{name}': the engine runs in bfloat16 or float32") from None


def build_from_config_dict(config_dict: dict):
    arch = resolve(config_dict)
    cfg = arch.parse_config(config_dict)
    return arch.build(cfg)


def tensor_specs_for(config):
    """The tensors a model of this configuration declares (no GPU needed)."""
    return build_from_config_dict(config.to_dict()).tensor_specs()


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0"):
    """Read config.json, pick the model by its architecture name, check and bind the weights."""
    model = build_from_config_dict(read_config_json(model_dir))
    ckpt = Checkpoint(model_dir)
    try:
        model.load(ckpt, Runtime(torch.device(device), parse_dtype(dtype)))
    finally:
        ckpt.close()
    return model


def random_model(config, seed: int = 0, std: float = 0.02, norm_sigma: float = 0.0, dtype="bfloat16",
                 device="cuda:0", weights_dtype: torch.dtype | None = None):
    """A model of `config` with seeded random weights made on the device, without a file."""
    model = build_from_config_dict(config.to_dict())
    rt = Runtime(torch.device(device), parse_dtype(dtype))
    src = RandomWeights(model.tensor_specs(), seed, std, norm_sigma, weights_dtype or torch.bfloat16, rt.device)
    model.load(src, rt)
    return model
