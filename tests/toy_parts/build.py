"""Builds tests/toy_parts/libtoy_parts.so from toy_parts.hip with hipcc for gfx950, against the
library's public header (picolm_amd/csrc/engine.h) and nothing else of the library's sources; the
one symbol it calls (picolm_set_error_message) is found in libpicolm_hip.so, which is loaded first."""
from __future__ import annotations

import ctypes
import hashlib
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SRC = os.path.join(HERE, "toy_parts.hip")
HEADER_DIR = os.path.join(ROOT, "picolm_amd", "csrc")


def _hash() -> str:
    h = hashlib.sha256()
    for p in (SRC, os.path.join(HEADER_DIR, "engine.h")):
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _targets():
    out = [HERE]
    out.append(os.path.join(tempfile.gettempdir(), f"picolm_amd-{os.getuid()}", "toy_parts"))
    return out


def build() -> str:
    from picolm_amd.csrc import build as lib_build
    hipcc = lib_build._hipcc()
    flags = [f for f in lib_build.FLAGS]
    last = None
    for d in _targets():
        try:
            os.makedirs(d, exist_ok=True)
            lib = os.path.join(d, "libtoy_parts.so")
            r = subprocess.run([hipcc, *flags, "-shared", "-I", HEADER_DIR, SRC, "-o", lib + ".tmp"], capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError("hipcc failed on toy_parts.hip:\n" + lib_build._filter(r.stdout + r.stderr))
            os.replace(lib + ".tmp", lib)
            with open(lib + ".hash", "w") as f:
                f.write(_hash())
            return lib
        except OSError as e:
            last = e
    raise RuntimeError(f"cannot write libtoy_parts.so: {last}")


def load() -> ctypes.CDLL:
    from picolm_amd import kernels
    kernels.lib()               # its symbols first, globally
    want = _hash()
    for d in _targets():
        lib = os.path.join(d, "libtoy_parts.so")
        try:
            with open(lib + ".hash") as f:
                if f.read().strip() == want:
                    return ctypes.CDLL(lib)
        except OSError:
            continue
    print("[toy_parts] building libtoy_parts.so", file=sys.stderr, flush=True)
    return ctypes.CDLL(build())
