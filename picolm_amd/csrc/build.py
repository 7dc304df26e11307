"""Builds and loads libpicolm_hip.so: the hand-written gfx950 kernels behind a C ABI.

The library is compiled with hipcc from the .hip files next to this one, one object per
file in parallel, and kept in-tree (picolm_amd/csrc/libpicolm_hip.so).  `load()` uses the
built library when its recorded source hash matches the sources and builds otherwise; a
first call in a fresh checkout therefore compiles, printing a line per file meanwhile.
When the tree cannot be written the build goes to a per-user folder under the system's
temporary directory.  There is no fallback: without the library the engine does not run.
"""
from __future__ import annotations

import concurrent.futures
import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libpicolm_hip.so"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    # packed FP32 instructions are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


class BuildError(RuntimeError):
    pass


def sources() -> list[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _headers() -> list[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for f in sources() + _headers():
        h.update(f.encode())
        with open(os.path.join(HERE, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.exists(c):
            return c
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _say(msg: str) -> None:
    print(f"[picolm_amd build] {msg}", file=sys.stderr, flush=True)


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        with tempfile.NamedTemporaryFile(dir=d):
            pass
        return True
    except OSError:
        return False


def _out_dirs() -> tuple[str, str]:
    """(folder of the library, folder of the objects)."""
    if _writable(HERE) and _writable(os.path.join(HERE, "_build")):
        return HERE, os.path.join(HERE, "_build")
    d = os.path.join(tempfile.gettempdir(), f"picolm_amd-{os.getuid()}", source_hash()[:16])
    os.makedirs(d, exist_ok=True)
    return d, d


def _filter(text: str) -> str:
    return "\n".join(l for l in text.splitlines() if "not a recognized feature for this target" not in l)


def _compile_one(hipcc: str, src: str, obj: str) -> tuple[str, float]:
    t0 = time.time()
    cmd = [hipcc, *FLAGS, "-I", HERE, "-c", os.path.join(HERE, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise BuildError(f"hipcc failed on {src}:\n{_filter(r.stdout + r.stderr)}")
    return src, time.time() - t0


def build(verbose: bool = True, jobs: int | None = None) -> str:
    """Compile every kernel source for gfx950 and link the library; returns its path."""
    hipcc = _hipcc()
    lib_dir, obj_dir = _out_dirs()
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16)
    if verbose:
        _say(f"compiling {len(srcs)} kernel files for {ARCH} with {jobs} jobs into {lib_dir}")
    objs = [os.path.join(obj_dir, s[:-4] + ".o") for s in srcs]
    t0 = time.time()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futs = [pool.submit(_compile_one, hipcc, s, o) for s, o in zip(srcs, objs)]
        pending = set(futs)
        while pending:
            done, pending = concurrent.futures.wait(pending, timeout=20)
            for f in done:
                src, dt = f.result()
                if verbose:
                    _say(f"  {src} compiled in {dt:.1f}s")
            if pending and verbose and not done:
                _say(f"  still compiling {len(pending)} files ({time.time() - t0:.0f}s)")
    lib = os.path.join(lib_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise BuildError(f"link failed:\n{_filter(r.stdout + r.stderr)}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(source_hash())
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.1f}s")
    return lib


def _built_library() -> str | None:
    want = source_hash()
    for d in (HERE, os.path.join(tempfile.gettempdir(), f"picolm_amd-{os.getuid()}", want[:16])):
        lib = os.path.join(d, LIB_NAME)
        try:
            with open(lib + ".hash") as f:
                if f.read().strip() == want and os.path.exists(lib):
                    return lib
        except OSError:
            continue
    return None


_LIB = None


def load() -> ctypes.CDLL:
    """The loaded library; builds it first if no current build exists."""
    global _LIB
    if _LIB is None:
        path = _built_library() or build()
        try:
            # (its symbols are visible to libraries loaded later: a part with kernels of its own, built
            # elsewhere, may call the error channel)
            _LIB = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        except OSError as e:
            raise BuildError(f"cannot load {path}: {e}") from None
    return _LIB


if __name__ == "__main__":
    build()
