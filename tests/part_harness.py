"""Runs one part of a layer alone inside the engine's step: a program that looks the given input
rows up (they are the rows of an embedding table, and a step's "tokens" are row numbers), lets
the part emit its operations, and returns the rows of a chosen buffer as the step's "logits".
The glue (a cast of float rows to the compute dtype, a buffer of zeros, the read-out) are called
operations written here in Python, so that nothing but the part under test is the library's."""
from __future__ import annotations

import numpy as np
import torch

from picolm_amd.cache import CacheSpec, KVGroupSpec, StateGroupSpec
from picolm_amd.engine import program as P
from picolm_amd.engine.native import NativeEngine
from picolm_amd.parts.base import CacheBinding, Runtime, Workspace, on_stream, rows_view

DEV = torch.device("cuda:0")


class PartEngine:
    def __init__(self, dtype: torch.dtype, rows: np.ndarray, emit, requests=(None, None), parts=(), n_slots: int = 4,
                 max_tokens: int = 1024, max_seq_len: int = 512, read_rows: int = P.ROWS_STEP):
        """rows [N, D]: every input row the steps will bring.  emit(builder, x, self) -> (buffer to
        read, its width): x is the float buffer [T, D] of the step's input rows.  requests: the
        (KVRequest, StateRequest) of the part, for the one cache entry.  parts: what to bind and
        prepare before emitting."""
        self.dtype, self.runtime = dtype, Runtime(DEV, dtype)
        self.ws = Workspace(DEV)
        N, D = rows.shape
        kv_req, st_req = requests
        for p in parts:
            p.bind_runtime(self.runtime, self.ws)
            if hasattr(p, "prepare"):
                p.prepare(self.runtime, max_seq_len)
        b = P.ProgramBuilder(dtype)
        self.builder = b
        x = b.buffer("x", D, torch.float32)
        b.binding = CacheBinding((0, 0) if kv_req else None, (0, 0) if st_req else None, True)
        # the table is padded to the width of the read-out below, which is not known yet: emit first
        marker = len(b.ops)
        out, width = emit(b, x, self)
        V = max(N, width)
        table = torch.zeros(V, D, dtype=torch.float32)
        table[:N] = torch.from_numpy(np.ascontiguousarray(rows)).float()
        self.table = table.to(DEV)
        embed = P.ProgramBuilder(dtype)
        embed.embed(self.table, x)
        b.ops.insert(marker, embed.ops[0])
        b.keep.append(self.table)
        self.width = width
        if out == "logits":                     # the part under test writes logits itself
            self.width = V = max(V, width)
        else:
            out_dtype = b.buffer_dtype(out)
            logits = b.buffer("logits", V, torch.float32, P.ROWS_WANTED)

            def read(view):
                with on_stream(view):
                    n_src = view.n_wanted if read_rows == P.ROWS_WANTED else view.n_tokens
                    src = rows_view(view.inp, n_src, view.in_row_bytes, out_dtype, DEV)
                    dst = rows_view(view.out, view.n_wanted, view.out_row_bytes, torch.float32, DEV)
                    if read_rows == P.ROWS_STEP:
                        want = rows_view(view.want_rows, 1, 4 * view.n_wanted, torch.int32, DEV)[0].long()
                        src = src[want]
                    dst[:, :width] = src[:, :width].float()
            b.call(read, out=logits, inp=out, rows=P.ROWS_WANTED)
            b.logits_buffer = logits
        spec = CacheSpec([KVGroupSpec(1, kv_req.n_kv_heads, kv_req.head_dim, kv_req.window, kv_req.v_head_dim)] if kv_req else [],
                         [StateGroupSpec(1, tuple(st_req.shape), st_req.dtype)] if st_req else [])
        self.vocab = V
        self.engine = NativeEngine(b.finish(V, spec), max_tokens, max_seq_len, n_slots, DEV)

    def cast(self, b, x: int, width: int, rows: int = P.ROWS_STEP, name: str = "h") -> int:
        """A buffer that holds the float rows of `x` (every row, or the wanted ones) in the compute dtype."""
        h = b.buffer(name, width, self.dtype, rows)
        dtype = self.dtype

        def run(view):
            with on_stream(view):
                src = rows_view(view.inp, view.n_tokens, view.in_row_bytes, torch.float32, DEV)
                if rows == P.ROWS_WANTED:
                    src = src[rows_view(view.want_rows, 1, 4 * view.n_wanted, torch.int32, DEV)[0].long()]
                rows_view(view.out, view.rows, view.out_row_bytes, dtype, DEV).copy_(src.to(dtype))
        b.call(run, out=h, inp=x, rows=rows)
        return h

    def zeros(self, b, width: int, name: str = "res") -> int:
        """A float buffer of the step's rows, zeroed by an operation."""
        r = b.buffer(name, width, torch.float32)

        def run(view):
            with on_stream(view):
                rows_view(view.out, view.n_tokens, view.out_row_bytes, torch.float32, DEV).zero_()
        b.call(run, out=r)
        return r

    def alloc(self, n: int):
        return [self.engine.slot_alloc() for _ in range(n)]

    def step(self, slots, row_ids, want=None) -> np.ndarray:
        """Sequence i brings the input rows row_ids[i]; returns the read buffer's rows [wanted, width]
        (default: every row)."""
        if want is None:
            want = [list(range(len(r))) for r in row_ids]
        out = self.engine.step(list(slots), [list(map(int, r)) for r in row_ids], want)
        return out[:, :self.width].double().cpu().numpy()
