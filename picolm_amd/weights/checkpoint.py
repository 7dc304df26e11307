"""A model folder's tensors by name, and the check of a model's needs against them.

picolm binds Llama tensors by their checkpoint names (picolm/safetensors.c:242-277), looks
a `model.language_model.` name up as `model.` too (:170-183), checks presence on layer 0
only (:509-512) and never checks a shape.  Here every tensor a model declares is checked,
and all faults are reported together in one `WeightsError`.

Storage policy: bfloat16 stays bfloat16, 32-bit floats stay 32-bit, integer tables become
int32.  The engine has no float16 arithmetic (picolm keeps such tensors as they are,
picolm/safetensors.c:163-164): in the 32-bit runtime a float16 tensor is widened to float32,
which is exact; in the bfloat16 runtime it is rounded to bfloat16, which drops three bits.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile

_RENAMES = (("model.language_model.", "model."),)
# buffers that older checkpoints of this family carry and that are no parameters: picolm binds
# tensors by name and never looks at the rest (picolm/safetensors.c:242-277)
_IGNORED_SUFFIXES = ("rotary_emb.inv_freq",)


class WeightsError(ValueError):
    """Lists every missing, unexpected and mis-shaped tensor of a checkpoint at once."""

    def __init__(self, source, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)      # (name, expected, found)
        self.wrong_dtype = list(wrong_dtype)      # (name, found)
        lines = [f"{source}: the checkpoint does not fit the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} expected {list(e)} found {list(f)}" for n, e, f in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  unsupported dtype ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n} is {d}" for n, d in self.wrong_dtype))
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class TensorSpec:
    """What a part needs from the checkpoint: a name, a shape, and whether it may be absent."""
    name: str
    shape: tuple
    optional: bool = False
    kind: str = "float"          # "float" or "int"
    init: str | None = "normal"  # random-weights mode: "normal", "ones", or None (not written)


def canonical_name(name: str) -> str:
    for old, new in _RENAMES:
        if name.startswith(old):
            return new + name[len(old):]
    return name


def stored_dtype(dtype: torch.dtype, kind: str = "float", runtime_dtype: torch.dtype | None = None) -> torch.dtype | None:
    """The dtype a tensor is kept in by a runtime of `runtime_dtype`, or None if the engine
    cannot hold it."""
    if kind == "int":
        return torch.int32 if dtype in (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8) else None
    if dtype == torch.float16:
        return torch.float32 if runtime_dtype == torch.float32 else torch.bfloat16
    if dtype == torch.bfloat16:
        return torch.bfloat16
    if dtype == torch.float32:
        return torch.float32
    return None


class Checkpoint:
    """The tensors of a model folder: `model.safetensors`, or shards named by
    `model.safetensors.index.json` (`weight_map`: tensor name -> file name)."""

    def __init__(self, model_dir: str):
        self.source = model_dir
        self._files: list[SafetensorsFile] = []
        self._where: dict[str, tuple] = {}        # canonical name -> (file, stored name)
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.isfile(single):
            paths = [single]
        elif os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as f:
                wm = json.load(f).get("weight_map", {})
            paths = [os.path.join(model_dir, p) for p in sorted(set(wm.values()))]
        else:
            raise SafetensorsError(f"{model_dir}: no model.safetensors and no model.safetensors.index.json")
        for p in paths:
            sf = SafetensorsFile(p)
            self._files.append(sf)
            for n in sf.names():
                c = canonical_name(n)
                if c in self._where:
                    raise SafetensorsError(f"{p}: tensor '{c}' is stored twice")
                self._where[c] = (sf, n)

    def names(self):
        return list(self._where)

    def metadata(self) -> dict:
        """What the files' headers carry beside tensors (`__metadata__`), all files together."""
        out = {}
        for sf in self._files:
            out.update({str(k): v for k, v in sf.metadata.items()})
        return out

    def info(self, name):
        sf, n = self._where[name]
        return sf.info(n)

    def tensor(self, name) -> torch.Tensor:
        sf, n = self._where[name]
        return sf.tensor(n)

    def close(self):
        for sf in self._files:
            sf.close()


class TensorDict:
    """The same interface over tensors already in memory (random weights, tests)."""

    def __init__(self, tensors: dict, source: str = "<memory>"):
        self.source = source
        self._t = dict(tensors)

    def names(self):
        return list(self._t)

    def info(self, name):
        t = self._t[name]
        return t.dtype, tuple(t.shape)

    def tensor(self, name):
        return self._t[name]

    def close(self):
        pass


def check_specs(source, specs: list[TensorSpec]) -> None:
    """Raise one WeightsError if `source` does not hold exactly what `specs` asks for."""
    wanted = {}
    for s in specs:
        if s.name in wanted and wanted[s.name].shape != tuple(s.shape):
            raise ValueError(f"two parts declare '{s.name}' with different shapes")
        wanted[s.name] = s
    have = set(source.names())
    missing = [n for n, s in wanted.items() if n not in have and not s.optional]
    unexpected = sorted(n for n in have - set(wanted) if not n.endswith(_IGNORED_SUFFIXES))
    wrong_shape, wrong_dtype = [], []
    for n, s in wanted.items():
        if n not in have:
            continue
        dtype, shape = source.info(n)
        if tuple(shape) != tuple(s.shape):
            wrong_shape.append((n, tuple(s.shape), tuple(shape)))
        if stored_dtype(dtype, s.kind) is None:
            wrong_dtype.append((n, str(dtype).replace("torch.", "")))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightsError(source.source, missing, unexpected, wrong_shape, wrong_dtype)


class WeightFetcher:
    """Hands checked tensors to the parts, in their kept dtype, on the target device."""

    def __init__(self, source, device, runtime_dtype: torch.dtype | None = None):
        self.source = source
        self.device = device
        self.runtime_dtype = runtime_dtype
        self._have = set(source.names())

    def has(self, name: str) -> bool:
        return name in self._have

    def get(self, name: str, kind: str = "float") -> torch.Tensor:
        t = self.source.tensor(name)
        dt = stored_dtype(t.dtype, kind, self.runtime_dtype)
        if dt is None:
            raise WeightsError(self.source.source, wrong_dtype=[(name, str(t.dtype))])
        t = t.to(device=self.device, non_blocking=False)
        return t if t.dtype == dt else t.to(dt)
