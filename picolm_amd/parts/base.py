"""What every part of a layer is: something that declares its tensors and its cache needs,
loads them, and acts on rows of a step.  No part knows which model it is in; its sizes and
constants are constructor parameters (picolm passes them as arguments too:
`rmsnorm(..., eps)` picolm/tensor.h:92, `rope(..., rope_type, half)` :102).

Interfaces
  Norm.forward(ctx, x[T,D] float32, rows=None)   -> h[n,D] in the compute dtype
  PositionEncoding.rotary_tables(ctx)            -> (cos, sin, style) or None, and
  PositionEncoding.apply(ctx, qkv, H, G, d)      in place, when it is not a rotation
  Mixer.forward(ctx, h[T,D], residual[T,D] f32)  adds its output into `residual`
  FeedForward.forward(ctx, h, residual)          adds its output into `residual`
  Block.forward(ctx, x[T,D] f32)                 the arrangement of the four above
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

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
    """Named scratch buffers that grow to the largest request and are reused by every
    layer; nothing is allocated in a step whose sizes were seen before."""

    def __init__(self, device):
        self.device = device
        self._bufs: dict[str, torch.Tensor] = {}
        self._flips: dict[str, int] = {}
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

    def zeros(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        """A buffer that is zero when first given out and that its users leave at zero (counters
        that a kernel resets itself)."""
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * dtype.itemsize
        buf = self._bufs.get(name)
        if buf is None or buf.numel() < nbytes:
            buf = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=self.device)
            self._bufs[name] = buf
        return buf[:nbytes].view(dtype).view(*shape)

    def flip(self, name: str) -> int:
        """0, 1, 0, 1, ... per name: for a pair of buffers used in turn."""
        self._flips[name] = 1 - self._flips.get(name, 1)
        return self._flips[name]

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


class StepContext:
    """What a part sees of the step it runs in."""

    def __init__(self, runtime: Runtime, batch, cache, workspace: Workspace):
        self.runtime = runtime
        self.batch = batch
        self.cache = cache
        self.ws = workspace
        self.binding: CacheBinding | None = None
        # the norm that will be applied to the residual stream after the running part has added to
        # it (set by the block; a Linear that adds into the stream may prepare it) and what such a
        # Linear prepared (picked up by whoever applies that norm next)
        self.norm_after: Norm | None = None
        self.prepared_norm: NormedRows | None = None
        self.norm_after_block: Norm | None = None      # set by the model for the block it calls

    @property
    def dtype(self) -> torch.dtype:
        return self.runtime.dtype

    def kv(self):
        """(k_pages, v_pages, page_table, ring_pages) of the running layer call."""
        gi, e = self.binding.kv
        g = self.cache.kv[gi]
        return g.k[e], g.v[e], g.table, g.ring_pages

    def kv_host(self):
        """(cache group index, the group's page table on the host) of the running layer call."""
        gi, _ = self.binding.kv
        return gi, self.cache.kv[gi].table_host

    def normed(self, norm: "Norm", x: torch.Tensor, part=None):
        """norm(x) for `part`: what a Linear prepared for this very norm and x if there is such a
        thing and the part passes it on to a Linear, else the norm's own kernel."""
        got, self.prepared_norm = self.prepared_norm, None
        if got is not None and got.norm is norm and got.x is x:
            return got if getattr(part, "takes_normed_rows", False) else got.tensor()
        return norm.forward(self, x)

    def state(self) -> torch.Tensor:
        """[n_slots, ...] state of the running layer call; index it with batch.seq_slot."""
        gi, e = self.binding.state
        return self.cache.state[gi][e]


class Part:
    """`emit`, where a part has it, appends the part's work to a launch program (engine/program.py)
    instead of running it: a model whose parts all have it is stepped by the library in one call.
    A part that only has `forward` is run from Python, and so is every model that contains one."""

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


class Norm(Part):
    def forward(self, ctx: StepContext, x: torch.Tensor, rows: torch.Tensor | None = None,
                n_rows: int | None = None) -> torch.Tensor:
        raise NotImplementedError

    def rms_parameters(self):
        """(float weights, eps) if this norm is y = x / sqrt(mean(x^2) + eps) * weights, which the
        products around it can compute between them (see NormedRows); None otherwise."""
        return None


class NormedRows:
    """norm(x) where the norm has not run as a kernel of its own.

    In a decode step a norm over a few rows is all launch latency, so the products around it
    share it: the Linear that finished x (adding into the residual stream) has left
    bf16(x * weights) and partial sums of x^2 (`prepared`), and the Linear that takes this object
    as its input multiplies its sums by 1 / sqrt(mean(x^2) + eps).  A part says with
    `takes_normed_rows = True` that it hands its input to a Linear unchanged; any other part is
    given `tensor()`, which runs the norm's own kernel on x."""

    def __init__(self, ctx: StepContext, norm: Norm, x: torch.Tensor, prepared=None):
        self.ctx, self.norm, self.x = ctx, norm, x
        self.prepared = prepared            # (h bf16 [T, D], ssq f32 [parts, 16]) or None
        self._tensor = None

    @property
    def shape(self):
        return self.x.shape

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.forward(self.ctx, self.x)
        return self._tensor


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


class FeedForward(Part):
    def forward(self, ctx: StepContext, h: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError


class Block(Part):
    mixer: Mixer

    def forward(self, ctx: StepContext, x: torch.Tensor) -> None:
        raise NotImplementedError
