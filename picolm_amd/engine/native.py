"""The Python face of the engine in libpicolm_hip.so (csrc/engine.h): a launch program goes in,
slots, steps and generation come out as single calls.  Everything a step needs lives in the
library (the books of the cache, the step's index arrays, the workspace, recorded decode steps);
this file only converts arguments and wraps the memory the library hands back as tensors.
"""
from __future__ import annotations

import ctypes
from ctypes import byref, c_int32, c_int64, c_void_p

import numpy as np
import torch

from .. import kernels
from ..cache import CacheError, CacheFull, window_ring_pages
from ..kernels import device_view
from . import program as P
from .errors import StepError

_declared = False


def _lib():
    global _declared
    lib = kernels.lib()
    if not _declared:
        P.declare(lib)
        _declared = True
    return lib


def _raise(rc: int, failures=None):
    if failures:            # a called Python operation raised: that exception, not its summary
        exc = failures.pop()
        del failures[:]
        raise exc
    msg = kernels.lib().picolm_last_error().decode("utf-8", "replace")
    if rc == P.ERR_STEP:
        raise StepError(msg)
    if rc == P.ERR_CACHE_FULL:
        raise CacheFull(msg)
    if rc == P.ERR_CACHE:
        raise CacheError(msg)
    raise kernels.KernelError(msg)


def _i32(values) -> np.ndarray:
    return np.ascontiguousarray(values, dtype=np.int32)


class _SlotCount:
    def __init__(self, engine):
        self._e = engine
        self.n_slots = engine.info(1)

    @property
    def n_free(self) -> int:
        return self._e.info(2)


class _KVEntries:
    """keys [entry][page][G][64][d] and values [entry][page][G][d][64] of one cache group, as the
    library keeps them."""

    def __init__(self, engine, group: int, spec, dtype, device):
        k, v, n = c_void_p(), c_void_p(), c_int64()
        rc = _lib().picolm_engine_kv_entry(engine.handle, group, 0, byref(k), byref(v), byref(n))
        if rc:
            _raise(rc)
        G, d = spec.n_kv_heads, spec.head_dim
        self.spec = spec
        self.ring_pages = min(window_ring_pages(spec.window), engine.info(5)) if spec.window > 0 else engine.info(5)
        self.k = device_view(k.value, (spec.n_entries, n.value, G, kernels.PAGE_TOKENS, d), dtype, device, engine._handle)
        self.v = device_view(v.value, (spec.n_entries, n.value, G, spec.value_dim, kernels.PAGE_TOKENS), dtype, device, engine._handle)


class EngineCache:
    """What generation and the tests ask of a cache, answered by the library's books."""

    def __init__(self, engine, cache_spec, dtype, device):
        self._e = engine
        self.spec = cache_spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_seq_len = engine.info(0)
        self.n_slots = engine.info(1)
        self.max_pages = engine.info(5)
        self.slots = _SlotCount(engine)
        self.kv = [_KVEntries(engine, gi, g, dtype, device) for gi, g in enumerate(cache_spec.kv_groups)]
        self.state = [self._state_entries(gi, g) for gi, g in enumerate(cache_spec.state_groups)]

    def _state_entries(self, group: int, spec) -> torch.Tensor:
        """[entry][slot][...] of one state group, as the library keeps it."""
        ptr, nbytes = c_void_p(), c_int64()
        rc = _lib().picolm_engine_state_entry(self._e.handle, group, 0, byref(ptr), byref(nbytes))
        if rc:
            _raise(rc)
        return device_view(ptr.value, (spec.n_entries, self.n_slots, *spec.shape), spec.dtype, self.device, self._e._handle)

    def length(self, slot: int) -> int:
        return max(self._e.length(slot), 0)

    def free_tokens(self) -> int:
        return self._e.info(3)

    def bytes(self) -> int:
        """Bytes of the keys, values and per-sequence state (the engine's other device memory,
        workspace and page tables, is in `engine.info(6)`)."""
        return self._e.info(9)

    @property
    def version(self) -> int:
        return self._e.info(7)


class _Handle:
    """Owns the engine in the library.  Tensors over the engine's memory keep it (and so that
    memory) alive: logits or a cache view that outlive their session stay readable."""

    def __init__(self, value):
        self.value = value

    def close(self) -> None:
        if self.value:
            _lib().picolm_engine_destroy(self.value)
            self.value = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class NativeEngine:
    def __init__(self, built: P.BuiltProgram, max_tokens: int, max_seq_len: int, n_slots: int | None, device,
                 graphs: bool = True, host_only: bool = False, time_ops: bool = False):
        self.program = built                      # keeps the weights and tables alive
        self.device = torch.device(device)
        self.vocab_size = built.struct.vocab_size
        flags = (0 if graphs else P.ENGINE_NO_GRAPHS) | (P.ENGINE_HOST_ONLY if host_only else 0) | (P.ENGINE_TIME_OPS if time_ops else 0)
        h = c_void_p()
        rc = _lib().picolm_engine_create(byref(built.struct), int(max_tokens), int(max_seq_len), int(n_slots or 0), flags,
                                         byref(h))
        if rc:
            _raise(rc)
        self._handle = _Handle(h)
        self.host_only = host_only
        self._views: dict = {}

    def _stream(self):
        return None if self.host_only else kernels._stream()

    @property
    def handle(self):
        return self._handle.value

    def close(self) -> None:
        """Destroys the engine now; tensors over its memory must not be used afterwards."""
        self._views.clear()
        self._handle.close()

    # -- books -----------------------------------------------------------------------------
    def info(self, what: int) -> int:
        return int(_lib().picolm_engine_info(self.handle, what))

    def slot_alloc(self) -> int:
        s = c_int32()
        rc = _lib().picolm_engine_slot_alloc(self.handle, byref(s), self._stream())
        if rc:
            _raise(rc)
        return s.value

    def slot_free(self, slot: int) -> None:
        rc = _lib().picolm_engine_slot_free(self.handle, int(slot))
        if rc:
            _raise(rc)

    def length(self, slot: int) -> int:
        return _lib().picolm_engine_slot_length(self.handle, int(slot))

    def slot_pages(self, group: int, slot: int) -> list[int]:
        out = np.zeros(max(self.info(5), 1), dtype=np.int32)
        n = _lib().picolm_engine_slot_pages(self.handle, group, slot, out.ctypes.data, len(out))
        if n < 0:
            _raise(n)
        return out[:n].tolist()

    def free_pages(self, group: int) -> int:
        return _lib().picolm_engine_free_pages(self.handle, group)

    def kv_pages(self, group: int) -> int:
        """Pages that a cache group has in all."""
        n = c_int64()
        rc = _lib().picolm_engine_kv_entry(self.handle, group, 0, None, None, byref(n))
        if rc:
            _raise(rc)
        return n.value

    def state_bytes_per_slot(self, group: int) -> int:
        n = c_int64()
        rc = _lib().picolm_engine_state_entry(self.handle, group, 0, None, byref(n))
        if rc:
            _raise(rc)
        return n.value

    def recorded_steps(self) -> int:
        return self.info(4)

    def op_times(self) -> dict:
        """GPU milliseconds since the last call by class of operation (an engine made with time_ops)."""
        ms = (ctypes.c_double * 4)()
        rc = _lib().picolm_engine_op_times(self.handle, ms)
        if rc:
            _raise(rc)
        return {"other": ms[0], "products": ms[1], "head": ms[2], "attention": ms[3]}

    def step_array(self, name: str) -> np.ndarray:
        n = _lib().picolm_engine_step_array(self.handle, name.encode(), None, 0)
        if n < 0:
            _raise(n)
        out = np.zeros(max(n, 1), dtype=np.int32)
        _lib().picolm_engine_step_array(self.handle, name.encode(), out.ctypes.data, n)
        return out[:n]

    # -- steps -----------------------------------------------------------------------------
    def _logits(self, ptr, rows: int) -> torch.Tensor:
        key = (ptr, rows)
        t = self._views.get(key)
        if t is None:
            if len(self._views) >= 256:
                self._views.clear()
            t = self._views[key] = device_view(ptr, (rows, self.vocab_size), torch.float32, self.device, self._handle)
        return t

    def step(self, slots, new_tokens, want=None) -> torch.Tensor | None:
        """As Session.step; None from an engine without device memory."""
        n = len(slots)
        if not (len(new_tokens) == n and (want is None or len(want) == n)):
            raise StepError("slots, tokens and wanted rows differ in length")
        if n == 0:
            raise StepError("a step needs at least one sequence")
        n_new = _i32([len(t) for t in new_tokens])
        flat = np.concatenate([np.asarray(t, dtype=np.int64).reshape(-1) for t in new_tokens]) if n_new.sum() else np.zeros(0, np.int64)
        if flat.size and (flat.min() < 0 or flat.max() >= self.vocab_size):
            bad = int(flat[(flat < 0) | (flat >= self.vocab_size)][0])
            raise StepError(f"token id {bad} is outside the vocabulary of {self.vocab_size}")
        tokens = _i32(flat)
        sl = _i32(list(slots))
        counts = idx = None
        if want is not None:
            counts = _i32([len(w) for w in want])
            idx = _i32([j for w in want for j in w]) if counts.sum() else np.zeros(1, np.int32)
        logits, rows = c_void_p(), c_int32()
        rc = _lib().picolm_engine_step(self.handle, n, sl.ctypes.data, n_new.ctypes.data, tokens.ctypes.data,
                                       counts.ctypes.data if counts is not None else None,
                                       idx.ctypes.data if idx is not None else None, byref(logits), byref(rows), self._stream())
        if rc:
            _raise(rc, self.program.failures)
        if not logits.value:
            return None if rows.value else torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        return self._logits(logits.value, rows.value)

    def step_device_tokens(self, slots, tokens: torch.Tensor) -> torch.Tensor:
        sl = _i32(list(slots))
        logits = c_void_p()
        rc = _lib().picolm_engine_step_device_tokens(self.handle, len(sl), sl.ctypes.data, tokens.data_ptr(), byref(logits),
                                                     kernels._stream())
        if rc:
            _raise(rc, self.program.failures)
        return self._logits(logits.value, len(sl))

    def generate(self, prompts, max_new_tokens: int, params, stop_ids=(), batch_size: int = 64,
                 prefill_step_tokens: int | None = None):
        """The library's own generation loop; returns (tokens of each request, finish reasons)."""
        if prefill_step_tokens is not None:
            rc = _lib().picolm_engine_set_prefill_step_tokens(self.handle, int(prefill_step_tokens))
            if rc:
                _raise(rc)
        n = len(prompts)
        lens = _i32([len(p) for p in prompts])
        flat = _i32(np.concatenate([np.asarray(p, dtype=np.int64) for p in prompts])) if n and lens.sum() else np.zeros(1, np.int32)
        stops = _i32(list(stop_ids)) if len(stop_ids) else np.zeros(1, np.int32)
        out = np.zeros((max(n, 1), max(max_new_tokens, 1)), dtype=np.int32)
        counts = np.zeros(max(n, 1), dtype=np.int32)
        finish = np.zeros(max(n, 1), dtype=np.int32)
        sp = P.Sampling(params.temperature, params.top_k, params.top_p, params.min_p, int(params.seed) & ((1 << 64) - 1))
        rc = _lib().picolm_engine_generate(self.handle, n, flat.ctypes.data, lens.ctypes.data, int(max_new_tokens), byref(sp),
                                           stops.ctypes.data, len(stop_ids), int(batch_size), out.ctypes.data, counts.ctypes.data,
                                           finish.ctypes.data, kernels._stream())
        if rc:
            _raise(rc, self.program.failures)
        reasons = {0: "", 1: "stop", 2: "length", 3: "capacity"}
        return [out[i, :counts[i]].tolist() for i in range(n)], [reasons[int(f)] for f in finish[:n]]
