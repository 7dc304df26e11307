"""Reading and writing the safetensors container.

Layout (what picolm/csafetensors.c:775-893 parses): 8 bytes little-endian header length,
a JSON object {name: {dtype, shape, data_offsets:[begin,end]}, "__metadata__": {...}},
then the bytes.  A file is mapped, never read whole; a tensor is a view into the map.
Offsets and sizes are checked against the file (the check picolm/csafetensors.c:1239-1276
has but its loader never calls).
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import torch


class SafetensorsError(ValueError):
    pass


_DTYPES = {
    "F32": torch.float32,
    "BF16": torch.bfloat16,
    "F16": torch.float16,
    "I32": torch.int32,
    "I64": torch.int64,
    "F64": torch.float64,
    "U8": torch.uint8,
    "I8": torch.int8,
    "I16": torch.int16,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


class SafetensorsFile:
    """One mapped file; `entries[name] = (dtype_name, shape, begin, end)`."""

    def __init__(self, path: str):
        self.path = path
        try:
            size = os.path.getsize(path)
        except OSError:
            raise SafetensorsError(f"{path}: no such file") from None
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header")
        self._file = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._file.read(8))
        if hlen > _MAX_HEADER or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds the file ({size} bytes)")
        try:
            header = json.loads(self._file.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not an object")
        self.metadata = header.pop("__metadata__", None) or {}
        self.data_start = 8 + hlen
        data_len = size - self.data_start
        self.entries: dict[str, tuple] = {}
        for name, info in header.items():
            try:
                dt, shape, (b, e) = info["dtype"], [int(s) for s in info["shape"]], info["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed entry for '{name}'") from None
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: '{name}' has dtype {dt}, which is not supported")
            if any(s < 0 for s in shape):
                raise SafetensorsError(f"{path}: '{name}' has a negative dimension {shape}")
            want = _numel(shape) * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if not (0 <= b <= e <= data_len) or e - b != want:
                raise SafetensorsError(
                    f"{path}: '{name}' {dt}{shape} needs {want} bytes but its offsets are [{b}, {e}) "
                    f"in a data section of {data_len}")
            self.entries[name] = (dt, tuple(shape), int(b), int(e))
        self._map = None

    def _mapped(self):
        if self._map is None:
            # ACCESS_COPY: private pages, so tensors over the map are writable without
            # touching the file.
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_COPY)
        return self._map

    def names(self):
        return list(self.entries)

    def info(self, name):
        dt, shape, _, _ = self.entries[name]
        return _DTYPES[dt], shape

    def tensor(self, name) -> torch.Tensor:
        dt, shape, b, e = self.entries[name]
        dtype = _DTYPES[dt]
        n = _numel(shape)
        if n == 0:
            return torch.empty(shape, dtype=dtype)
        t = torch.frombuffer(self._mapped(), dtype=dtype, count=n, offset=self.data_start + b)
        return t.view(shape)

    def close(self):
        # Tensors handed out keep the map alive through the buffer protocol; only the
        # descriptor is released here.
        self._file.close()


def write_safetensors(path: str, tensors, metadata: dict | None = None) -> None:
    """Write `tensors` (dict or iterable of (name, CPU tensor)) in the order given.

    The header is written first from shapes alone, so tensors may be produced one at a
    time by a generator that is run twice: pass a callable returning a fresh iterable.
    """
    make = tensors if callable(tensors) else (lambda: tensors.items() if isinstance(tensors, dict) else tensors)
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, t in make():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"'{name}': dtype {t.dtype} cannot be written")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t in make():
            t = t.detach().contiguous().cpu()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
