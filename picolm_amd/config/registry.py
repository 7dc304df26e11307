"""One registry from an architecture's name (config.json `architectures[0]`) to its model.

picolm has no such table: it sniffs the architecture from substrings of GGUF metadata
(picolm/model_gguf.c:729-751) and from which tensors exist.  Here an architecture is an
entry with two callables: one that types the config.json, one that builds the model's
parts from the typed configuration.

An architecture that lives outside the package registers itself when its module is imported.
The command line, trace replay and every other entry point import the modules named in the
environment variable PICOLM_ARCHITECTURES (comma-separated, found on sys.path like any module)
before they look a name up, so that such an architecture needs no change to the package.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable

from .llama import ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[dict], object]      # dict of config.json -> typed configuration
    build: Callable[..., object]                # (config, runtime) -> DecoderModel


_REGISTRY: dict[str, Architecture] = {}


def register_architecture(name: str, parse_config, build, *, replace: bool = False) -> Architecture:
    _load_builtin()
    if name in _REGISTRY and not replace:
        raise ConfigError(f"architecture '{name}' is already registered")
    arch = Architecture(name, parse_config, build)
    _REGISTRY[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _REGISTRY.pop(name, None)


_BUILTIN_LOADED = False


def _load_builtin() -> None:
    """The architectures that ship with the library register themselves when imported."""
    global _BUILTIN_LOADED
    if not _BUILTIN_LOADED:
        _BUILTIN_LOADED = True
        from ..engine import llama  # noqa: F401


_OUTSIDE_LOADED = False


def _load_all() -> None:
    """Before a name is looked up: the library's own architectures and those of the modules that
    PICOLM_ARCHITECTURES names (which import the package, so they wait until it is whole)."""
    global _OUTSIDE_LOADED
    _load_builtin()
    if not _OUTSIDE_LOADED:
        _OUTSIDE_LOADED = True
        import_architecture_modules(os.environ.get("PICOLM_ARCHITECTURES", ""))


def import_architecture_modules(names: str) -> list[str]:
    """Imports the comma-separated modules, each of which calls `register_architecture`; returns
    their names.  A module that cannot be imported is a configuration error that names it."""
    import importlib
    done = []
    for name in (n.strip() for n in names.split(",")):
        if not name:
            continue
        try:
            importlib.import_module(name)
        except Exception as exc:
            raise ConfigError(f"PICOLM_ARCHITECTURES: cannot import '{name}': {type(exc).__name__}: {exc}") from exc
        done.append(name)
    return done


def known_architectures() -> list[str]:
    _load_all()
    return sorted(_REGISTRY)


def architecture_name(config_dict: dict) -> str:
    archs = config_dict.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        return str(archs[0])
    if isinstance(archs, str):
        return archs
    raise ConfigError("architectures: missing; config.json must name its architecture "
                      f"(known: {', '.join(known_architectures())})")


def resolve(config_dict: dict) -> Architecture:
    _load_all()
    name = architecture_name(config_dict)
    if name not in _REGISTRY:
        raise ConfigError(f"architectures: '{name}' is not registered "
                          f"(known: {', '.join(known_architectures())})")
    return _REGISTRY[name]


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json") if os.path.isdir(model_dir) else model_dir
    try:
        with open(path, "r", encoding="utf-8") as f:
            return json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no config.json") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not JSON ({e})") from None
