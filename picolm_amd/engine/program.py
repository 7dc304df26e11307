"""A model as a launch program: the flat list of operations over named row buffers that the
parts of a model emit once and that the engine in libpicolm_hip.so walks at every step
(csrc/engine.h).  The structures here mirror that header field by field.

A part runs inside the engine through `emit(builder, ...)`: it appends its operations and names
the buffers it needs.  The built-in parts are compositions of the engine's own operations
(embedding, product with its epilogue and the norms around it, attention over a cache entry); a
part with kernels of its own, or one written in Python, appends a *called* operation
(`ProgramBuilder.call`): a function that the engine hands the running step to.
"""
from __future__ import annotations

import ctypes
import traceback
from ctypes import CFUNCTYPE, POINTER, Structure, c_float, c_int, c_int32, c_int64, c_uint64, c_void_p
from dataclasses import dataclass

import torch

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}
OP_EMBED, OP_RMSNORM, OP_LINEAR, OP_ATTENTION, OP_CALL = 1, 2, 3, 4, 5
ROWS_STEP, ROWS_WANTED = 0, 1
ENGINE_NO_GRAPHS, ENGINE_HOST_ONLY, ENGINE_TIME_OPS = 1, 2, 4
ERR_STEP, ERR_CACHE_FULL, ERR_CACHE, ERR_DEVICE = -10, -11, -12, -13
CALL_RECORDABLE, CALL_KV, CALL_ATTENDS, CALL_STATE = 1, 2, 4, 8


class Buffer(Structure):
    _fields_ = [("row_bytes", c_int32), ("rows", c_int32), ("dtype", c_int32)]


class StepView(Structure):
    """picolm_step_view: what a called operation sees of the running step."""
    _fields_ = [
        ("struct_bytes", c_int32), ("dtype", c_int32),
        ("n_seq", c_int32), ("n_tokens", c_int32), ("n_wanted", c_int32),
        ("is_decode", c_int32), ("every_row_wanted", c_int32), ("recording", c_int32),
        ("slots", POINTER(c_int32)), ("pos0", POINTER(c_int32)), ("n_new", POINTER(c_int32)),
        ("seq_slot", c_void_p), ("seq_pos0", c_void_p), ("seq_nnew", c_void_p), ("cu_seqlens", c_void_p),
        ("tok_pos", c_void_p), ("tok_seq", c_void_p), ("tokens", c_void_p), ("want_rows", c_void_p),
        ("rows", c_int32),
        ("inp", c_void_p), ("out", c_void_p), ("extra", c_void_p * 4),
        ("in_row_bytes", c_int32), ("out_row_bytes", c_int32), ("extra_row_bytes", c_int32 * 4),
        ("k_pages", c_void_p), ("v_pages", c_void_p), ("page_table", c_void_p),
        ("n_pages", c_int32), ("max_pages", c_int32), ("ring_pages", c_int32), ("n_kv_heads", c_int32),
        ("head_dim", c_int32), ("v_head_dim", c_int32), ("window", c_int32), ("kv_writes", c_int32),
        ("write_pages", c_void_p),
        ("chunk_list", c_void_p), ("n_chunks", c_int32), ("pages_per_chunk", c_int32), ("most_chunks", c_int32),
        ("partial", c_void_p), ("counters", c_void_p),
        ("tile_seq", c_void_p), ("tile_q0", c_void_p), ("n_tiles", c_int32), ("tile_rows", c_int32),
        ("state", c_void_p), ("state_bytes_per_slot", c_int64), ("n_slots", c_int32),
        ("stream", c_void_p),
    ]


CALL_FN = CFUNCTYPE(c_int, c_void_p, POINTER(StepView))


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
        ("call", c_void_p), ("call_user", c_void_p), ("call_flags", c_int32),
        ("state_group", c_int32), ("state_entry", c_int32), ("extra", c_int32 * 4),
        ("tile_rows", c_int32), ("partial_floats", c_int32),
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


class NormRef:
    """An RMSNorm as the operations around it see it: float weights on the device and eps."""

    def __init__(self, weight: torch.Tensor, eps: float):
        self.weight, self.eps = weight, float(eps)


@dataclass(frozen=True)
class Rows:
    """The rows a part takes as its input: those of `buffer` as they are, or, with `norm`, the
    RMSNorm of the float rows in buffer `x`, for which `buffer` is the place if someone has to
    write them out (a product computes such a norm on its way in, and in decode steps shares it
    with the product before; `ProgramBuilder.materialize` runs it as an operation of its own)."""
    buffer: int
    norm: NormRef | None = None
    x: int = -1


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
        self.keep = []                        # tensors and callbacks whose addresses the operations hold
        self.binding = None                   # the cache binding of the layer call being emitted
        self.logits_buffer = -1
        self.failures: list = []              # exceptions that called Python operations raised, newest last

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

    def buffer_dtype(self, index: int) -> torch.dtype:
        return torch.float32 if self._specs[index][2] == F32 else torch.bfloat16

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

    def rmsnorm(self, norm: NormRef, x: int, out: int, rows: int = ROWS_STEP) -> None:
        self.ops.append(Op(kind=OP_RMSNORM, rows=rows, inp=x, out=out, weight=self._ptr(norm.weight), k=norm.weight.shape[0],
                           eps=norm.eps))

    def materialize(self, src: Rows, rows: int = ROWS_STEP) -> int:
        """The buffer that holds `src`'s rows, after running the norm they are the result of, if any,
        as an operation of its own: for parts that do not hand their input to a product."""
        if src.norm is not None:
            self.rmsnorm(src.norm, src.x, src.buffer, rows)
        return src.buffer

    def linear(self, weight: torch.Tensor, src, out: int, epilogue: int, rows: int = ROWS_STEP,
               out_norm: NormRef | None = None, out_norm_when: int = 0) -> None:
        """out (=, +=, = silu-gated) rows W^T; `src` is a buffer or `Rows`.  out_norm: the RMSNorm
        that meets `out` next (with the accumulating epilogue), which the product may prepare;
        out_norm_when = 1: only in steps that want every row."""
        if not isinstance(src, Rows):
            src = Rows(int(src))
        op = Op(kind=OP_LINEAR, rows=rows, inp=src.buffer, out=out, weight=self._ptr(weight), weight_dt=_DT[weight.dtype],
                n=weight.shape[0], k=weight.shape[1], epilogue=epilogue)
        if src.norm is not None:
            op.in_norm_weight, op.in_norm_eps, op.in_norm_x = self._ptr(src.norm.weight), src.norm.eps, src.x
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

    def call(self, fn, out: int, inp: int = -1, extra=(), rows: int = ROWS_STEP, user=None, recordable: bool = False,
             uses_kv: bool = False, attends: bool = False, uses_state: bool = False, tile_rows: int = 0,
             partial_floats: int = 0) -> None:
        """An operation of the caller's.  `fn`: a C function `int (*)(void* user, const
        picolm_step_view*)` as a ctypes function pointer or address (with `user`, an address or a
        ctypes object that is kept alive), or a Python callable taking the `StepView`; it queues
        its work on the view's stream.  `out` (required), `inp`, `extra`: the buffers it is handed.
        `recordable`: what it queues depends on device memory only, so a decode step that holds it
        may be recorded once and replayed (a Python callable that says so must not allocate GPU
        memory while the stream records).  uses_kv / uses_state: it is handed the cache entry / the
        state entry of the layer call being emitted; attends: also the decode step's work list and,
        with tile_rows, the prefill step's tiles."""
        if len(extra) > 4:
            raise ValueError("a called operation names at most four buffers beside its input and output")
        b = self.binding
        if uses_kv and (b is None or b.kv is None):
            raise ValueError("a called operation that uses keys and values needs the cache entry of its layer call")
        if uses_state and (b is None or b.state is None):
            raise ValueError("a called operation that uses state needs the state entry of its layer call")
        if callable(fn) and not isinstance(fn, ctypes._CFuncPtr):
            fn = self._trampoline(fn)
        if isinstance(fn, ctypes._CFuncPtr):
            self.keep.append(fn)
            address = ctypes.cast(fn, c_void_p).value
        else:
            address = int(fn)
        if user is not None and not isinstance(user, int):
            self.keep.append(user)
            user = ctypes.addressof(user)
        flags = ((CALL_RECORDABLE if recordable else 0) | (CALL_KV if uses_kv else 0) | (CALL_ATTENDS if attends else 0) |
                 (CALL_STATE if uses_state else 0))
        op = Op(kind=OP_CALL, rows=rows, inp=inp, out=out, call=address, call_user=user, call_flags=flags,
                tile_rows=tile_rows, partial_floats=partial_floats)
        op.extra = (c_int32 * 4)(*(list(extra) + [-1] * (4 - len(extra))))
        if uses_kv:
            op.kv_group, op.kv_entry, op.kv_writes = b.kv[0], b.kv[1], int(b.writes)
        if uses_state:
            op.state_group, op.state_entry = b.state
        self.ops.append(op)

    def _trampoline(self, fn):
        """`fn(view)` as a C function; what it raises fails the step and is kept for the caller of
        the step."""
        failures = self.failures

        def entry(_user, view):
            try:
                if view.contents.struct_bytes != ctypes.sizeof(StepView):
                    raise RuntimeError(f"the library's step view has {view.contents.struct_bytes} bytes, this module's "
                                       f"{ctypes.sizeof(StepView)}: picolm_amd/engine/program.py and csrc/engine.h differ")
                fn(view.contents)
                return 0
            except BaseException as exc:        # nothing may cross the C frames between here and the step's caller
                del failures[:]
                failures.append(exc)
                from .. import kernels
                message = "".join(traceback.format_exception_only(type(exc), exc)).strip()
                kernels.lib().picolm_set_error_message(f"a called operation raised {message}".encode("utf-8", "replace"))
                return ERR_STEP
        return CALL_FN(entry)

    def finish(self, vocab_size: int, cache_spec) -> "BuiltProgram":
        if self.logits_buffer < 0:
            raise ValueError("the program writes no logits")
        return BuiltProgram(self, vocab_size, cache_spec)


class BuiltProgram:
    """The ctypes form of a program, with everything its pointers refer to kept alive."""

    def __init__(self, b: ProgramBuilder, vocab_size: int, cache_spec):
        self.keep = list(b.keep)
        self.failures = b.failures
        self.ops = (Op * len(b.ops))(*b.ops)
        self.buffers = (Buffer * len(b._specs))(*[Buffer(*s) for s in b._specs])
        kv = [KVGroup(g.n_entries, g.n_kv_heads, g.head_dim, g.window, g.v_head_dim) for g in cache_spec.kv_groups]
        st = [StateGroup(g.n_entries, g.bytes_per_slot) for g in cache_spec.state_groups]
        self.kv_groups = (KVGroup * max(len(kv), 1))(*kv)
        self.state_groups = (StateGroup * max(len(st), 1))(*st)
        self.struct = Program(dtype=_DT[b.dtype], vocab_size=vocab_size, ops=self.ops, n_ops=len(b.ops), buffers=self.buffers,
                              n_buffers=len(b._specs), logits_buffer=b.logits_buffer, kv_groups=self.kv_groups,
                              n_kv_groups=len(kv), state_groups=self.state_groups, n_state_groups=len(st))
        self.buffer_names = dict(b._buffers)
        self.n_ops = len(b.ops)
        self.recordable = all(op.kind != OP_CALL or op.call_flags & CALL_RECORDABLE for op in b.ops)


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
    lib.picolm_set_error_message.argtypes = [ctypes.c_char_p]
    lib.picolm_set_error_message.restype = None
    for name in ("create", "slot_alloc", "slot_free", "slot_length", "step", "step_device_tokens", "generate", "kv_entry",
                 "state_entry", "slot_pages", "free_pages", "step_array"):
        getattr(lib, "picolm_engine_" + name).restype = ctypes.c_int
