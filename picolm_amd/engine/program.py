"""A model as a launch program: the flat list of operations over named row buffers that the
parts of a model emit once and that the engine in libpicolm_hip.so walks at every step
(csrc/engine.h).  The structures here mirror that header field by field.

A part that can run inside the engine has `emit(builder, ...)`; it appends its operations and
names the buffers it needs.  A model whose parts all have it is stepped by the library in one
call; any other model is stepped part by part from Python (`DecoderModel.step`).
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int32, c_int64, c_uint64, c_void_p

import torch

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}
OP_EMBED, OP_RMSNORM, OP_LINEAR, OP_ATTENTION = 1, 2, 3, 4
ROWS_STEP, ROWS_WANTED = 0, 1
ENGINE_NO_GRAPHS, ENGINE_HOST_ONLY, ENGINE_TIME_OPS = 1, 2, 4
ERR_STEP, ERR_CACHE_FULL, ERR_CACHE, ERR_DEVICE = -10, -11, -12, -13


class Buffer(Structure):
    _fields_ = [("row_bytes", c_int32), ("rows", c_int32), ("dtype", c_int32)]


class Op(Structure):
    _fields_ = [
        ("kind", c_int32), ("rows", c_int32), ("inp", c_int32), ("out", c_int32),
        ("weight", c_void_p), ("weight_dt", c_int32), ("n", c_int32), ("k", c_int32), ("epilogue", c_int32),
        ("eps", c_float),
        ("in_norm_weight", c_void_p), ("in_norm_eps", c_float), ("in_norm_x", c_int32),
        ("out_norm_weight", c_void_p), ("out_norm_eps", c_float), ("out_norm_when", c_int32),
        ("n_heads", c_int32), ("n_kv_heads", c_int32), ("head_dim", c_int32), ("window", c_int32),
        ("scale", c_float),
        ("cos_table", c_void_p), ("sin_table", c_void_p), ("rope_style", c_int32), ("table_positions", c_int32),
        ("kv_group", c_int32), ("kv_entry", c_int32), ("kv_writes", c_int32), ("q_buffer", c_int32),
    ]


class KVGroup(Structure):
    _fields_ = [("n_entries", c_int32), ("n_kv_heads", c_int32), ("head_dim", c_int32), ("window", c_int32),
                ("v_head_dim", c_int32)]


class StateGroup(Structure):
    _fields_ = [("n_entries", c_int32), ("bytes_per_slot", c_int64)]


class Program(Structure):
    _fields_ = [
        ("dtype", c_int32), ("vocab_size", c_int32),
        ("ops", POINTER(Op)), ("n_ops", c_int32),
        ("buffers", POINTER(Buffer)), ("n_buffers", c_int32),
        ("logits_buffer", c_int32),
        ("kv_groups", POINTER(KVGroup)), ("n_kv_groups", c_int32),
        ("state_groups", POINTER(StateGroup)), ("n_state_groups", c_int32),
    ]


class Sampling(Structure):
    _fields_ = [("temperature", c_float), ("top_k", c_int32), ("top_p", c_float), ("min_p", c_float), ("seed", c_uint64)]


class CannotEmit(Exception):
    """A part that has no operations of the engine's for what it does: its model is stepped part by
    part from Python."""


class NormRef:
    """An RMSNorm as the operations around it see it: float weights on the device and eps."""

    def __init__(self, weight: torch.Tensor, eps: float):
        self.weight, self.eps = weight, float(eps)


class ProgramBuilder:
    """Collects the operations and buffers that parts emit.  Buffers are named; two parts that
    ask for the same name share the memory (a layer's scratch is the next layer's), and the
    widest request sizes it."""

    def __init__(self, dtype: torch.dtype, host_only: bool = False):
        self.dtype = dtype
        self.host_only = host_only            # a program for an engine without device memory: addresses are not used
        self.ops: list[Op] = []
        self._buffers: dict[str, int] = {}
        self._specs: list[list] = []          # [row_bytes, rows, dtype]
        self.keep = []                        # tensors whose addresses the operations hold
        self.binding = None                   # the cache binding of the layer call being emitted
        self.logits_buffer = -1

    def buffer(self, name: str, width: int, dtype: torch.dtype, rows: int = ROWS_STEP) -> int:
        row_bytes = int(width) * dtype.itemsize
        i = self._buffers.get(name)
        if i is None:
            i = self._buffers[name] = len(self._specs)
            self._specs.append([row_bytes, rows, _DT[dtype]])
        else:
            spec = self._specs[i]
            if spec[1] != rows or spec[2] != _DT[dtype]:
                raise ValueError(f"buffer '{name}' is asked for with two kinds of rows or two dtypes")
            spec[0] = max(spec[0], row_bytes)
        return i

    def _ptr(self, t: torch.Tensor | None):
        if t is None:
            return None
        if not (t.is_cuda or self.host_only) or not t.is_contiguous():
            raise ValueError("an operation's weights and tables lie contiguous in GPU memory")
        self.keep.append(t)
        return t.data_ptr()

    def embed(self, table: torch.Tensor, out: int) -> None:
        self.ops.append(Op(kind=OP_EMBED, rows=ROWS_STEP, out=out, weight=self._ptr(table), weight_dt=_DT[table.dtype],
                           n=table.shape[0], k=table.shape[1]))

    def linear(self, weight: torch.Tensor, inp: int, out: int, epilogue: int, rows: int = ROWS_STEP,
               in_norm: NormRef | None = None, in_norm_x: int = -1, out_norm: NormRef | None = None,
               out_norm_when: int = 0) -> None:
        op = Op(kind=OP_LINEAR, rows=rows, inp=inp, out=out, weight=self._ptr(weight), weight_dt=_DT[weight.dtype],
                n=weight.shape[0], k=weight.shape[1], epilogue=epilogue)
        if in_norm is not None:
            op.in_norm_weight, op.in_norm_eps, op.in_norm_x = self._ptr(in_norm.weight), in_norm.eps, in_norm_x
        if out_norm is not None:
            op.out_norm_weight, op.out_norm_eps, op.out_norm_when = self._ptr(out_norm.weight), out_norm.eps, out_norm_when
        self.ops.append(op)

    def attention(self, inp: int, q_buffer: int, out: int, n_heads: int, n_kv_heads: int, head_dim: int, window: int,
                  scale: float, tables) -> None:
        b = self.binding
        if b is None or b.kv is None:
            raise ValueError("an attention operation needs the cache entry of its layer call")
        op = Op(kind=OP_ATTENTION, rows=ROWS_STEP, inp=inp, out=out, q_buffer=q_buffer, n_heads=n_heads, n_kv_heads=n_kv_heads,
                head_dim=head_dim, window=window, scale=scale, kv_group=b.kv[0], kv_entry=b.kv[1], kv_writes=int(b.writes))
        if tables is not None:
            cos, sin, style = tables
            op.cos_table, op.sin_table, op.rope_style, op.table_positions = self._ptr(cos), self._ptr(sin), style, cos.shape[0]
        self.ops.append(op)

    def finish(self, vocab_size: int, cache_spec) -> "BuiltProgram":
        if self.logits_buffer < 0:
            raise ValueError("the program writes no logits")
        return BuiltProgram(self, vocab_size, cache_spec)


class BuiltProgram:
    """The ctypes form of a program, with everything its pointers refer to kept alive."""

    def __init__(self, b: ProgramBuilder, vocab_size: int, cache_spec):
        self.keep = list(b.keep)
        self.ops = (Op * len(b.ops))(*b.ops)
        self.buffers = (Buffer * len(b._specs))(*[Buffer(*s) for s in b._specs])
        kv = [KVGroup(g.n_entries, g.n_kv_heads, g.head_dim, g.window, g.v_head_dim) for g in cache_spec.kv_groups]
        st = []
        for g in cache_spec.state_groups:
            n = g.dtype.itemsize
            for s in g.shape:
                n *= int(s)
            st.append(StateGroup(g.n_entries, n))
        self.kv_groups = (KVGroup * max(len(kv), 1))(*kv)
        self.state_groups = (StateGroup * max(len(st), 1))(*st)
        self.struct = Program(dtype=_DT[b.dtype], vocab_size=vocab_size, ops=self.ops, n_ops=len(b.ops), buffers=self.buffers,
                              n_buffers=len(b._specs), logits_buffer=b.logits_buffer, kv_groups=self.kv_groups,
                              n_kv_groups=len(kv), state_groups=self.state_groups, n_state_groups=len(st))
        self.buffer_names = dict(b._buffers)
        self.n_ops = len(b.ops)


def declare(lib) -> None:
    """Argument and result types of the engine's entry points."""
    E = c_void_p
    I32P = POINTER(c_int32)
    lib.picolm_engine_create.argtypes = [POINTER(Program), c_int64, c_int32, c_int32, c_int32, POINTER(E)]
    lib.picolm_engine_destroy.argtypes = [E]
    lib.picolm_engine_destroy.restype = None
    lib.picolm_engine_slot_alloc.argtypes = [E, I32P, c_void_p]
    lib.picolm_engine_slot_free.argtypes = [E, c_int32]
    lib.picolm_engine_slot_length.argtypes = [E, c_int32]
    lib.picolm_engine_step.argtypes = [E, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_void_p), I32P,
                                       c_void_p]
    lib.picolm_engine_step_device_tokens.argtypes = [E, c_int32, c_void_p, c_void_p, POINTER(c_void_p), c_void_p]
    lib.picolm_engine_generate.argtypes = [E, c_int32, c_void_p, c_void_p, c_int32, POINTER(Sampling), c_void_p, c_int32,
                                           c_int32, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.picolm_engine_set_prefill_step_tokens.argtypes = [E, c_int32]
    lib.picolm_engine_set_prefill_step_tokens.restype = ctypes.c_int
    lib.picolm_engine_op_times.argtypes = [E, c_void_p]
    lib.picolm_engine_op_times.restype = ctypes.c_int
    lib.picolm_engine_info.argtypes = [E, c_int32]
    lib.picolm_engine_info.restype = c_int64
    lib.picolm_engine_kv_entry.argtypes = [E, c_int32, c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64)]
    lib.picolm_engine_state_entry.argtypes = [E, c_int32, c_int32, POINTER(c_void_p), POINTER(c_int64)]
    lib.picolm_engine_slot_pages.argtypes = [E, c_int32, c_int32, c_void_p, c_int32]
    lib.picolm_engine_free_pages.argtypes = [E, c_int32]
    lib.picolm_engine_step_array.argtypes = [E, ctypes.c_char_p, c_void_p, c_int32]
    for name in ("create", "slot_alloc", "slot_free", "slot_length", "step", "step_device_tokens", "generate", "kv_entry",
                 "state_entry", "slot_pages", "free_pages", "step_array"):
        getattr(lib, "picolm_engine_" + name).restype = ctypes.c_int
