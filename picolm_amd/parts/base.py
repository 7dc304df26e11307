"""What every part of a layer is: something that declares its tensors and its cache needs,
loads them, and puts its work into a launch program.  No part knows which model it is in; its
sizes and constants are constructor parameters (picolm passes them as arguments too:
`rmsnorm(..., eps)` picolm/tensor.h:92, `rope(..., rope_type, half)` :102).

A part joins a model's program through `emit` (engine/program.py).  The built-in parts emit the
engine's own operations.  A part that only defines `forward`, which runs its kernels (or torch
operators) on the tensors it is handed, inherits an `emit` that wraps `forward` into a called
operation: the engine hands it the running step, and it sees the step's rows, its cache entry and
its state as tensors over the engine's memory.

Interfaces (a new part implements `forward`, or `emit`, or both)
  Norm.forward(ctx, x[T,D] float32, rows=None, n_rows=None) -> h[n,D] in the compute dtype
  Norm.emit(b, x, rows) -> Rows                  the norm of buffer x as a part's input
  PositionEncoding.rotary_tables()               -> (cos, sin, style) or None, and
  PositionEncoding.apply(ctx, qkv, H, G, d)      in place, when it is not a rotation
  Mixer.forward(ctx, h[T,D], residual[T,D] f32)  adds its output into `residual`
  Mixer.emit(b, src: Rows, x, out_norm, out_norm_when)
  FeedForward.forward / .emit                    the same
  Block.emit(b, x, after, after_when)            the arrangement of the four above
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import kernels
from ..weights import TensorSpec


@dataclass
class Runtime:
    """Where and in which precision a model runs."""
    device: torch.device
    dtype: torch.dtype              # torch.bfloat16: serving precision; torch.float32: true 32-bit

    @property
    def is_f32(self) -> bool:
        return self.dtype == torch.float32


class Workspace:
    """Named scratch buffers for parts that run from Python: they grow to the largest request and
    are reused; nothing is allocated in a step whose sizes were seen before."""

    def __init__(self, device):
        self.device = device
        self._bufs: dict[str, torch.Tensor] = {}
        self._views: dict[tuple, tuple] = {}      # (name, shape, dtype) -> (buffer, view of it)

    def get(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        key = (name, tuple(shape), dtype)
        hit = self._views.get(key)
        if hit is not None and hit[0] is self._bufs.get(name):
            return hit[1]                       # the same request as before: the same view
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * dtype.itemsize
        buf = self._bufs.get(name)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=self.device)
            self._bufs[name] = buf
        view = buf[:nbytes].view(dtype).view(*shape)
        if len(self._views) >= 4096:            # (a long run of steps of ever new sizes)
            self._views.clear()
        self._views[key] = (buf, view)
        return view

    def bytes(self) -> int:
        return sum(b.numel() for b in self._bufs.values())


@dataclass(frozen=True)
class KVRequest:
    """A mixer's need for keys and values of each token.  `head_dim` is the size of a key;
    `v_head_dim` that of a value where it differs (0: the same)."""
    n_kv_heads: int
    head_dim: int
    window: int = 0
    v_head_dim: int = 0

    def __post_init__(self):
        if self.v_head_dim == self.head_dim:        # one way to say "the same": requests compare equal
            object.__setattr__(self, "v_head_dim", 0)

    @property
    def value_dim(self) -> int:
        return self.v_head_dim or self.head_dim


@dataclass(frozen=True)
class StateRequest:
    """A mixer's need for a fixed-size tensor per sequence."""
    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass
class CacheBinding:
    """Where one layer call finds its cache: (group, entry) for each of its requests, and
    whether this call writes the entries or reads another call's."""
    kv: tuple | None = None          # (group index, entry index)
    state: tuple | None = None
    writes: bool = True


class StepArrays:
    """The running step as a part that runs from Python sees it: host lists per sequence and the
    engine's device arrays as int32 tensors (made when first asked for)."""

    _DEVICE = {"seq_slot": "n_seq", "seq_pos0": "n_seq", "seq_nnew": "n_seq", "tok_pos": "T", "tok_seq": "T", "tokens": "T",
               "want_rows": "n_want"}

    def __init__(self, view, device):
        self._view, self._device = view, device
        self.n_seq, self.T, self.n_want = view.n_seq, view.n_tokens, view.n_wanted
        self.is_decode = bool(view.is_decode)
        self.wants_every_row = bool(view.every_row_wanted)
        self.slots = view.slots[:self.n_seq]
        self.pos0 = view.pos0[:self.n_seq]
        self.n_new = view.n_new[:self.n_seq]
        self.max_new = max(self.n_new)
        self.max_len = max(p + n for p, n in zip(self.pos0, self.n_new))

    def __getattr__(self, name):
        if name == "cu_seqlens":
            n = self.n_seq + 1
        elif name in self._DEVICE:
            n = getattr(self, self._DEVICE[name])
        else:
            raise AttributeError(name)
        t = kernels.device_view(getattr(self._view, name), (max(n, 1),), torch.int32, self._device)[:n]
        setattr(self, name, t)
        return t

    def write_pages(self) -> torch.Tensor:
        """For every token of the step the physical page that takes its key and value (int32 [T])."""
        if not self._view.write_pages:
            raise ValueError("this layer call writes no keys and values")
        return kernels.device_view(self._view.write_pages, (self.T,), torch.int32, self._device)


class StepContext:
    """What a part that runs from Python sees of the step it runs in."""

    def __init__(self, runtime: Runtime, view, workspace: Workspace, state_request: StateRequest | None = None):
        self.runtime = runtime
        self.view = view
        self.ws = workspace
        self.batch = StepArrays(view, runtime.device)
        self.recording = bool(view.recording)
        self._state_request = state_request

    @property
    def dtype(self) -> torch.dtype:
        return self.runtime.dtype

    def kv(self):
        """(k_pages [pages, G, 64, d], v_pages [pages, G, dv, 64], page_table [slots, max_pages],
        ring_pages) of the running layer call."""
        v = self.view
        if not v.k_pages:
            raise ValueError("this part asked for no keys and values (cache_requests)")
        k = kernels.device_view(v.k_pages, (v.n_pages, v.n_kv_heads, kernels.PAGE_TOKENS, v.head_dim), self.dtype, self.runtime.device)
        vv = kernels.device_view(v.v_pages, (v.n_pages, v.n_kv_heads, v.v_head_dim, kernels.PAGE_TOKENS), self.dtype, self.runtime.device)
        table = kernels.device_view(v.page_table, (v.n_slots, v.max_pages), torch.int32, self.runtime.device)
        return k, vv, table, v.ring_pages

    @property
    def writes_cache(self) -> bool:
        return bool(self.view.kv_writes)

    def state(self) -> torch.Tensor:
        """[n_slots, ...] state of the running layer call; index it with batch.slots / batch.seq_slot."""
        v, rq = self.view, self._state_request
        if not v.state or rq is None:
            raise ValueError("this part asked for no state (cache_requests)")
        return kernels.device_view(v.state, (v.n_slots, *rq.shape), rq.dtype, self.runtime.device)


def rows_view(ptr, rows: int, row_bytes: int, dtype: torch.dtype, device) -> torch.Tensor:
    """A row buffer of the engine's as a tensor [rows, width]."""
    return kernels.device_view(ptr, (rows, row_bytes // dtype.itemsize), dtype, device)


def keeps_forward(part, cls) -> bool:
    """Whether `part` still does in `forward` what `cls.emit` emits: a subclass that changes
    `forward` and leaves `emit` alone has changed the work, and runs through `forward`."""
    t = type(part)
    return t.forward is cls.forward or t.emit is not cls.emit


def forward_is_graph_safe(part, method: str = "forward") -> bool:
    """Whether the class that defines the part's `forward` (or one derived from it) says
    `graph_safe = True` itself: a subclass that writes a `forward` of its own does not inherit the
    word of the class it changed."""
    for cls in type(part).__mro__:
        if cls.__dict__.get("graph_safe") is True:
            return True
        if method in cls.__dict__:
            return False
    return False


class Part:
    graph_safe = False      # True: what `forward` queues depends on device memory only and allocates nothing anew, so
                            # that a decode step which holds it can be recorded once and replayed

    def tensor_specs(self) -> list[TensorSpec]:
        return []

    def load(self, fetch, runtime: Runtime) -> None:
        pass

    def children(self) -> list["Part"]:
        return []

    def all_specs(self) -> list[TensorSpec]:
        out = list(self.tensor_specs())
        for c in self.children():
            out.extend(c.all_specs())
        return out

    def load_all(self, fetch, runtime: Runtime) -> None:
        self.load(fetch, runtime)
        for c in self.children():
            c.load_all(fetch, runtime)

    def bind_runtime(self, runtime: Runtime, workspace: Workspace) -> None:
        """Called before a model's program is emitted: where the part runs, and scratch memory
        for the parts that run from Python."""
        self._runtime, self._workspace = runtime, workspace
        for c in self.children():
            c.bind_runtime(runtime, workspace)

    def _context(self, view, state_request=None) -> StepContext:
        return StepContext(self._runtime, view, self._workspace, state_request)


class on_stream:
    """Runs the body with torch's current stream set to the stream of a step view (the engine
    records decode steps on a stream of its own)."""

    def __init__(self, view):
        self._raw = view.stream or 0
        self._guard = None

    def __enter__(self):
        if self._raw != (kernels._stream().value or 0):
            self._guard = torch.cuda.stream(torch.cuda.ExternalStream(self._raw))
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            self._guard.__exit__(*exc)


class Norm(Part):
    size: int

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: torch.Tensor | None = None,
                n_rows: int | None = None) -> torch.Tensor:
        raise NotImplementedError

    def emit(self, b, x: int, rows: int = 0):
        """This norm of the float rows in buffer `x` (of the step's rows, or with rows = 1 of the
        rows whose logits are wanted) as the input of the part that follows: a `Rows`."""
        from ..engine.program import ROWS_WANTED, Rows
        width = b._specs[x][0] // 4
        h = b.buffer("norm.final" if rows == ROWS_WANTED else "norm.out", width, b.dtype, rows)
        dtype = b.dtype

        def run(view):
            with on_stream(view):
                ctx = self._context(view)
                xt = rows_view(view.inp, view.n_tokens, view.in_row_bytes, torch.float32, ctx.runtime.device)
                out = rows_view(view.out, view.rows, view.out_row_bytes, dtype, ctx.runtime.device)
                if rows == ROWS_WANTED and not view.every_row_wanted:
                    y = self.forward(ctx, xt, rows=ctx.batch.want_rows, n_rows=view.n_wanted)
                else:
                    y = self.forward(ctx, xt)
                out[:, :y.shape[1]].copy_(y)
        b.call(run, out=h, inp=x, rows=rows, recordable=forward_is_graph_safe(self))
        return Rows(h)


class PositionEncoding(Part):
    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        pass

    def rotary_tables(self):
        return None

    def apply(self, ctx: StepContext, qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int) -> None:
        pass


class Mixer(Part):
    def cache_requests(self) -> tuple:
        """(KVRequest | None, StateRequest | None)"""
        return (None, None)

    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        pass

    def forward(self, ctx: StepContext, h: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += mixer(src) as operations of a launch program.  This one hands the step to `forward`."""
        _emit_forward(self, b, src, x, *self.cache_requests())


class FeedForward(Part):
    def forward(self, ctx: StepContext, h: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += ffn(src) as operations of a launch program.  This one hands the step to `forward`."""
        _emit_forward(self, b, src, x, None, None)


def _emit_forward(part, b, src, x: int, kv_request, state_request) -> None:
    h = b.materialize(src)
    h_dtype = b.buffer_dtype(h)

    def run(view):
        with on_stream(view):
            ctx = part._context(view, state_request)
            dev = ctx.runtime.device
            part.forward(ctx, rows_view(view.inp, view.n_tokens, view.in_row_bytes, h_dtype, dev),
                         rows_view(view.out, view.n_tokens, view.out_row_bytes, torch.float32, dev))
    b.call(run, out=x, inp=h, uses_kv=kv_request is not None, uses_state=state_request is not None,
           recordable=forward_is_graph_safe(part))


class Block(Part):
    mixer: Mixer

    def first_norm(self):
        """The norm this block applies to the residual stream on entry, if the block before may
        prepare it."""
        return None

    def forward(self, ctx: StepContext, x: torch.Tensor) -> None:
        raise NotImplementedError

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        """The block over the residual rows in buffer `x`.  This one hands the step to `forward`."""
        kv_request, state_request = self.mixer.cache_requests()

        def run(view):
            with on_stream(view):
                ctx = self._context(view, state_request)
                self.forward(ctx, rows_view(view.out, view.n_tokens, view.out_row_bytes, torch.float32, ctx.runtime.device))
        b.call(run, out=x, uses_kv=kv_request is not None, uses_state=state_request is not None,
               recordable=forward_is_graph_safe(self))
