"""Builds tests/c_client/tiny_llama_c from tiny_llama.c with the C compiler (C11, not HIP): a
client that sees the library through its two public headers (picolm_amd/csrc/engine.h, api.h) and
links libpicolm_hip.so and the HIP runtime."""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SRC = os.path.join(HERE, "tiny_llama.c")
HEADER_DIR = os.path.join(ROOT, "picolm_amd", "csrc")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def _hash() -> str:
    h = hashlib.sha256()
    for p in (SRC, os.path.join(HEADER_DIR, "engine.h"), os.path.join(HEADER_DIR, "api.h")):
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _targets():
    return [HERE, os.path.join(tempfile.gettempdir(), f"picolm_amd-{os.getuid()}", "c_client")]


def build(library: str | None = None) -> str:
    """Compiles and links against `library` (default: the library next to its sources)."""
    cc = os.environ.get("CC") or shutil.which("gcc") or shutil.which("cc") or shutil.which("clang")
    if not cc:
        raise RuntimeError("no C compiler found (looked at $CC, gcc, cc, clang)")
    lib_dir = os.path.dirname(library) if library else HEADER_DIR
    last = None
    for d in _targets():
        try:
            os.makedirs(d, exist_ok=True)
            exe = os.path.join(d, "tiny_llama_c")
            cmd = [cc, "-std=c11", "-O1", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROCM, "include"), "-I", HEADER_DIR,
                   SRC, "-o", exe + ".tmp", "-L", lib_dir, "-lpicolm_hip", "-L", os.path.join(ROCM, "lib"), "-lamdhip64", "-lm",
                   "-Wl,-rpath," + lib_dir, "-Wl,-rpath," + os.path.join(ROCM, "lib")]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError("the C compiler failed on tiny_llama.c:\n" + r.stdout + r.stderr)
            os.replace(exe + ".tmp", exe)
            with open(exe + ".hash", "w") as f:
                f.write(_hash())
            return exe
        except OSError as e:
            last = e
    raise RuntimeError(f"cannot write tiny_llama_c: {last}")


def binary(library: str) -> str:
    """The built client, built now if it is missing or older than its sources."""
    want = _hash()
    for d in _targets():
        exe = os.path.join(d, "tiny_llama_c")
        try:
            with open(exe + ".hash") as f:
                if f.read().strip() == want and os.path.exists(exe):
                    return exe
        except OSError:
            continue
    print("[c_client] building tiny_llama_c", file=sys.stderr, flush=True)
    return build(library)
