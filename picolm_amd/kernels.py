"""Python face of libpicolm_hip.so: each function checks its operands on the host (device,
dtype, shape, contiguity) and queues one hand-written gfx950 kernel on torch's current
stream.  There is no fallback: a missing library or a CPU tensor is an error.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from .csrc import build as _build

F32, BF16 = 0, 1
PAGE_TOKENS = 64
_DT = {torch.float32: F32, torch.bfloat16: BF16}

EPI_STORE, EPI_ACCUMULATE, EPI_SWIGLU = 0, 1, 2


class KernelError(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        l = _build.load()
        l.picolm_last_error.restype = ctypes.c_char_p
        for name in dir_entry_points():
            getattr(l, name).restype = c_int
        l.picolm_read_probe_bytes.restype = ctypes.c_size_t
        if l.picolm_abi_version() != 2:
            raise KernelError("libpicolm_hip.so has another ABI version; rebuild it")
        _lib = l
    return _lib


def dir_entry_points():
    return ["picolm_abi_version", "picolm_device_check", "picolm_embed", "picolm_gather_i32", "picolm_rmsnorm",
            "picolm_rope_kv_store", "picolm_gemm_generic",
            "picolm_attn_prefill_tile_rows", "picolm_attn_prefill_generic",
            "picolm_attn_decode_generic", "picolm_argmax", "picolm_argmax_scratch_floats", "picolm_sample", "picolm_sample_scratch_bytes", "picolm_gemm_skinny", "picolm_gemm_tiled", "picolm_gemm_tiled_splitk", "picolm_gemm_linked", "picolm_gemm_tiled_norm_parts", "picolm_kv_page_order",
            "picolm_attn_mfma_takes", "picolm_attn_prefill_mfma_heads", "picolm_attn_prefill_mfma_tile_tokens",
            "picolm_attn_prefill_mfma", "picolm_attn_decode_mfma", "picolm_attn_decode_rope_mfma", "picolm_attn_decode_mfma_waves", "picolm_read_probe", "picolm_mfma_probe",
            "picolm_linear", "picolm_linear_norm_rows", "picolm_linear_norm_parts", "picolm_linear_links_norms",
            "picolm_linear_medium_splits", "picolm_argmax_static", "picolm_argmax_static_max_floats"]


def _check(rc: int) -> None:
    if rc != 0:
        raise KernelError(lib().picolm_last_error().decode("utf-8", "replace"))


def require_device() -> None:
    """Fail loudly unless a gfx950 GPU and the kernel library are there."""
    if not torch.cuda.is_available():
        raise KernelError("no GPU: picolm_amd runs on an MI355X (gfx950) only and has no CPU path")
    _check(lib().picolm_device_check())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> c_void_p:
    """torch's current stream on the current device (asked for at every launch: a graph is
    recorded on a stream of its own)."""
    if _raw_stream is not None:           # the same handle without building a Stream object
        return c_void_p(_raw_stream(torch.cuda.current_device()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: torch.Tensor | None) -> c_void_p:
    return c_void_p(0) if t is None else c_void_p(t.data_ptr())


def _dev(name: str, t: torch.Tensor, dtype=None, dim=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: expected a GPU tensor")
    if not t.is_contiguous():
        raise KernelError(f"{name}: expected a contiguous tensor")
    if dtype is not None:
        ok = t.dtype in dtype if isinstance(dtype, (tuple, list)) else t.dtype == dtype
        if not ok:
            raise KernelError(f"{name}: dtype {t.dtype} is not {dtype}")
    if dim is not None and t.dim() != dim:
        raise KernelError(f"{name}: expected {dim} dimensions, got {tuple(t.shape)}")
    return t


def _i32(name, t, n=None):
    _dev(name, t, torch.int32)
    if n is not None and t.numel() < n:
        raise KernelError(f"{name}: holds {t.numel()} entries, {n} are needed")
    return t


class _DeviceMemory:
    """Memory that the library owns, for torch to look at (never to free).  `owner`: whatever must
    stay alive as long as a tensor over this memory does."""

    def __init__(self, ptr: int, nbytes: int, owner=None):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr, False), "version": 2}
        self.owner = owner


def device_view(ptr: int, shape, dtype: torch.dtype, device, owner=None) -> torch.Tensor:
    """A tensor over `ptr`, device memory that someone else owns."""
    n = dtype.itemsize
    for s in shape:
        n *= int(s)
    if n == 0 or not ptr:
        return torch.empty(tuple(shape), dtype=dtype, device=device)
    return torch.as_tensor(_DeviceMemory(ptr, n, owner), device=device).view(dtype).view(*shape)


def dt_of(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is neither float32 nor bfloat16") from None


# --------------------------------------------------------------------------------------------
def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> None:
    _dev("embed.table", table, (torch.float32, torch.bfloat16), 2)
    _i32("embed.tokens", tokens)
    _dev("embed.out", out, torch.float32, 2)
    T, D = out.shape
    if table.shape[1] != D or tokens.numel() < T:
        raise KernelError(f"embed: table {tuple(table.shape)}, tokens {tokens.numel()}, out {tuple(out.shape)} do not fit")
    _check(lib().picolm_embed(_ptr(table), dt_of(table), _ptr(tokens), _ptr(out), T, D, table.shape[0], _stream()))


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            rows: torch.Tensor | None = None) -> None:
    _dev("rmsnorm.x", x, torch.float32, 2)
    _dev("rmsnorm.weight", weight, torch.float32, 1)
    _dev("rmsnorm.out", out, (torch.float32, torch.bfloat16), 2)
    D = x.shape[1]
    n = out.shape[0]
    if weight.numel() != D or out.shape[1] != D:
        raise KernelError(f"rmsnorm: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)} do not fit")
    if rows is None:
        if n > x.shape[0]:
            raise KernelError("rmsnorm: more output rows than input rows")
    else:
        _i32("rmsnorm.rows", rows, n)
    _check(lib().picolm_rmsnorm(_ptr(x), _ptr(weight), _ptr(out), dt_of(out), _ptr(rows), n, D,
                                c_float(eps), _stream()))


def rope_kv_store(qkv, q_out, k_pages, v_pages, cos, sin, style: int, tok_pos, tok_page, H: int, G: int, d: int,
                  rows=None, n_rows: int | None = None) -> None:
    """Rotate q and k of every token row (or of `rows` only) and write k, v to the cache: token
    t goes to row tok_pos[t] % 64 of physical page tok_page[t]."""
    _dev("rope.qkv", qkv, torch.float32, 2)
    T = qkv.shape[0]
    if qkv.shape[1] != (H + 2 * G) * d:
        raise KernelError(f"rope: qkv has {qkv.shape[1]} columns, (H+2G)d = {(H + 2 * G) * d}")
    if q_out is None and k_pages is None:
        raise KernelError("rope: neither q nor the cache to write")
    if q_out is not None:
        _dev("rope.q_out", q_out, (torch.float32, torch.bfloat16), 2)
        if tuple(q_out.shape) != (T, H * d):
            raise KernelError(f"rope: q_out {tuple(q_out.shape)} is not {(T, H * d)}")
    if k_pages is not None:
        _check_pages("rope", k_pages, v_pages, q_out.dtype if q_out is not None else k_pages.dtype, G, d)
        _i32("rope.tok_page", tok_page, T)
    if cos is not None:
        _dev("rope.cos", cos, torch.float32, 2)
        _dev("rope.sin", sin, torch.float32, 2)
        if cos.shape[1] != d // 2 or sin.shape != cos.shape:
            raise KernelError(f"rope: tables {tuple(cos.shape)} do not have d/2 = {d // 2} columns")
    _i32("rope.tok_pos", tok_pos, T)
    n_launch = T
    if rows is not None:
        n_launch = rows.numel() if n_rows is None else n_rows
        _i32("rope.rows", rows, n_launch)
        if n_launch > T:
            raise KernelError("rope: more rows listed than there are")
    _check(lib().picolm_rope_kv_store(
        _ptr(qkv), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), dt_of(q_out if q_out is not None else k_pages), _ptr(cos), _ptr(sin), style,
        _ptr(tok_pos), _ptr(tok_page if k_pages is not None else None), n_launch, H, G, d, _ptr(rows), _stream()))


_page_orders: dict = {}


def kv_page_order(dtype: torch.dtype, d: int):
    """Where K[key][i] and V^T[i][key] lie within a group's part of a cache page: two int64
    tensors k_idx [64, d] and v_idx [d, 64] of element offsets.  Plain arrays, except in bfloat16
    pages of the head sizes that the matrix-core kernels take: those hold their 16-byte chunks
    in the order in which a wave loads them as MFMA operands."""
    key = (dtype, d)
    if key not in _page_orders:
        import numpy as np
        k_idx = np.empty(PAGE_TOKENS * d, np.int32)
        v_idx = np.empty(PAGE_TOKENS * d, np.int32)
        _check(lib().picolm_kv_page_order(_DT[dtype], d, k_idx.ctypes.data_as(c_void_p), v_idx.ctypes.data_as(c_void_p)))
        _page_orders[key] = (torch.from_numpy(k_idx.astype(np.int64)).reshape(PAGE_TOKENS, d),
                             torch.from_numpy(v_idx.astype(np.int64)).reshape(d, PAGE_TOKENS))
    return _page_orders[key]


def kv_pages_pack(k: torch.Tensor, v: torch.Tensor):
    """Pages given as plain arrays k [pages, G, 64, d], v [pages, G, d, 64] in the order the
    kernels keep them (same shapes and dtype)."""
    k_idx, v_idx = kv_page_order(k.dtype, k.shape[-1])
    kp, vp = torch.empty_like(k), torch.empty_like(v)
    kp.view(*k.shape[:2], -1)[..., k_idx.reshape(-1).to(k.device)] = k.reshape(*k.shape[:2], -1)
    vp.view(*v.shape[:2], -1)[..., v_idx.reshape(-1).to(v.device)] = v.reshape(*v.shape[:2], -1)
    return kp, vp


def kv_pages_unpack(k_pages: torch.Tensor, v_pages: torch.Tensor):
    """The kernels' pages as plain arrays k [pages, G, 64, d], v [pages, G, d, 64]."""
    k_idx, v_idx = kv_page_order(k_pages.dtype, k_pages.shape[-1])
    k = k_pages.reshape(*k_pages.shape[:2], -1)[..., k_idx.reshape(-1).to(k_pages.device)].view(k_pages.shape)
    v = v_pages.reshape(*v_pages.shape[:2], -1)[..., v_idx.reshape(-1).to(v_pages.device)].view(v_pages.shape)
    return k, v


def _check_pages(who, k_pages, v_pages, dtype, G, d):
    """keys [pages, G, PAGE, d]; values transposed [pages, G, d, PAGE]"""
    _dev(who + ".k_pages", k_pages, dtype, 4)
    _dev(who + ".v_pages", v_pages, dtype, 4)
    if tuple(k_pages.shape[1:]) != (G, PAGE_TOKENS, d):
        raise KernelError(f"{who}: k_pages {tuple(k_pages.shape)} is not [pages, {G}, {PAGE_TOKENS}, {d}]")
    if tuple(v_pages.shape[1:]) != (G, d, PAGE_TOKENS) or v_pages.shape[0] != k_pages.shape[0]:
        raise KernelError(f"{who}: v_pages {tuple(v_pages.shape)} is not [{k_pages.shape[0]}, {G}, {d}, {PAGE_TOKENS}]")


def gemm_generic(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int = EPI_STORE) -> None:
    """c = a @ w.T (store), c += a @ w.T (accumulate) or the gated form over interleaved rows of w."""
    M, N, K = _gemm_shapes(a, w, c, epilogue)
    _check(lib().picolm_gemm_generic(_ptr(a), dt_of(a), _ptr(w), dt_of(w), _ptr(c), dt_of(c), M, N, K,
                                     c_int64(K), c_int64(K), c_int64(c.shape[1]), epilogue, _stream()))


def _gemm_shapes(a, w, c, epilogue):
    _dev("gemm.a", a, (torch.float32, torch.bfloat16), 2)
    _dev("gemm.w", w, (torch.float32, torch.bfloat16), 2)
    _dev("gemm.c", c, (torch.float32, torch.bfloat16), 2)
    M, K = a.shape
    N = w.shape[0]
    n_out = N // 2 if epilogue == EPI_SWIGLU else N
    if w.shape[1] != K or tuple(c.shape) != (M, n_out):
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)} do not fit (epilogue {epilogue})")
    return M, N, K


def attn_prefill_tile_rows() -> int:
    return lib().picolm_attn_prefill_tile_rows()


def attn_prefill_generic(q, k_pages, v_pages, out, tile_seq, tile_q0, n_tiles, seq_slot, seq_pos0,
                         seq_nnew, cu_seqlens, page_table, ring_pages, H, G, d, window, scale) -> None:
    _attn_check(q, k_pages, v_pages, out, page_table, H, G, d)
    _i32("attn.tile_seq", tile_seq, n_tiles)
    _i32("attn.tile_q0", tile_q0, n_tiles)
    for nm, t in (("seq_slot", seq_slot), ("seq_pos0", seq_pos0), ("seq_nnew", seq_nnew), ("cu_seqlens", cu_seqlens)):
        _i32("attn." + nm, t)
    _check(lib().picolm_attn_prefill_generic(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), dt_of(q), _ptr(tile_seq), _ptr(tile_q0), n_tiles,
        _ptr(seq_slot), _ptr(seq_pos0), _ptr(seq_nnew), _ptr(cu_seqlens), _ptr(page_table),
        page_table.shape[1], ring_pages, H, G, d, window, c_float(scale), _stream()))


def _decode_check(q, partial, n_seq, chunk_list, n_chunks, pages_per_chunk, max_splits, seq_pos0, H, d) -> None:
    if max_splits > 1:
        _dev("attn.partial", partial, torch.float32)
        if partial.numel() < n_seq * H * max_splits * (d + 2):
            raise KernelError("attn_decode: the partial buffer is too small")
    if q.shape[0] < n_seq:
        raise KernelError("attn_decode: fewer query rows than sequences")
    if pages_per_chunk < 1 or max_splits < 1:
        raise KernelError(f"attn_decode: {pages_per_chunk} pages a chunk, {max_splits} chunks a sequence")
    _i32("attn.chunk_list", chunk_list, 8 * (n_chunks + 1))
    _i32("attn.seq_pos0", seq_pos0, n_seq)


def attn_decode_generic(q, k_pages, v_pages, out, partial, n_seq, chunk_list, n_chunks, pages_per_chunk,
                        max_splits, seq_pos0, page_table, ring_pages, H, G, d, window, scale) -> None:
    _attn_check(q, k_pages, v_pages, out, page_table, H, G, d)
    _decode_check(q, partial, n_seq, chunk_list, n_chunks, pages_per_chunk, max_splits, seq_pos0, H, d)
    _check(lib().picolm_attn_decode_generic(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(partial if max_splits > 1 else None), dt_of(q),
        n_seq, _ptr(chunk_list), n_chunks, pages_per_chunk, max_splits, _ptr(seq_pos0), _ptr(page_table),
        page_table.shape[1], ring_pages, H, G, d, window, c_float(scale), _stream()))


def _attn_check(q, k_pages, v_pages, out, page_table, H, G, d):
    _dev("attn.q", q, (torch.float32, torch.bfloat16), 2)
    _dev("attn.out", out, q.dtype, 2)
    if q.shape[1] != H * d or out.shape != q.shape:
        raise KernelError(f"attn: q {tuple(q.shape)} / out {tuple(out.shape)} are not [T, {H * d}]")
    _check_pages("attn", k_pages, v_pages, q.dtype, G, d)
    _dev("attn.page_table", page_table, torch.int32, 2)


def argmax_scratch_floats(n_rows: int, V: int) -> int:
    return lib().picolm_argmax_scratch_floats(n_rows, V)


def argmax(logits: torch.Tensor, out: torch.Tensor, scratch: torch.Tensor | None = None) -> None:
    """The first maximum of every row; `scratch` (float32, argmax_scratch_floats) is made if not given."""
    _dev("argmax.logits", logits, torch.float32, 2)
    n, V = logits.shape
    _i32("argmax.out", out, n)
    need = argmax_scratch_floats(n, V)
    if scratch is None:
        scratch = torch.empty(max(need, 1), dtype=torch.float32, device=logits.device)
    _dev("argmax.scratch", scratch, torch.float32)
    if scratch.numel() < need:
        raise KernelError(f"argmax: scratch holds {scratch.numel()} floats, {need} are needed")
    _check(lib().picolm_argmax(_ptr(logits), _ptr(out), n, V, c_int64(V), _ptr(scratch), _stream()))


SKINNY_MAX_M = 64


def gemm_skinny(a, w, c, epilogue: int = EPI_STORE, variant: int = 0) -> None:
    """bf16 x bf16 on the matrix cores for M <= 64 rows: weights streamed once from HBM."""
    M, N, K = _gemm_shapes(a, w, c, epilogue)
    _check(lib().picolm_gemm_skinny(_ptr(a), _ptr(w), _ptr(c), dt_of(c), M, N, K, c_int64(K), c_int64(K),
                                    c_int64(c.shape[1]), epilogue, variant, _stream()))


def gemm_tiled(a, w, c, epilogue: int = EPI_STORE, variant: int = 0) -> None:
    """bf16 x bf16 on the matrix cores, LDS-tiled, for many rows."""
    M, N, K = _gemm_shapes(a, w, c, epilogue)
    _check(lib().picolm_gemm_tiled(_ptr(a), _ptr(w), _ptr(c), dt_of(c), M, N, K, c_int64(K), c_int64(K),
                                   c_int64(c.shape[1]), epilogue, variant, _stream()))


SPLITK_WS_FLOATS = 8 << 20        # 32 MB of partial sums: splits * M * N may not exceed it
_splitk_ws: dict = {}


def splitk_workspace(device) -> torch.Tensor:
    """One buffer per GPU for the partial sums of products cut along K; kernels of one stream
    run in order, so they can share it."""
    key = torch.device(device).index or 0
    if key not in _splitk_ws:
        _splitk_ws[key] = torch.empty(SPLITK_WS_FLOATS, dtype=torch.float32, device=device)
    return _splitk_ws[key]


def gemm_tiled_splitk(a, w, c, epilogue: int, variant: int, splits: int) -> None:
    M, N, K = _gemm_shapes(a, w, c, epilogue)
    if splits > 1 and splits * M * N > SPLITK_WS_FLOATS:
        raise KernelError(f"gemm: {splits} splits of {M}x{N} exceed the workspace")
    ws = splitk_workspace(a.device) if splits > 1 else None
    _check(lib().picolm_gemm_tiled_splitk(_ptr(a), _ptr(w), _ptr(c), dt_of(c), M, N, K, c_int64(K), c_int64(K),
                                          c_int64(c.shape[1]), epilogue, variant, splits, _ptr(ws), _stream()))


def medium_gemm_splits(M: int, N: int, K: int) -> int:
    """Into how many parts along K a product of 17..64 rows is cut: its tiles hold 128 weight
    rows each, and every CU should have one."""
    return lib().picolm_linear_medium_splits(M, N, K)


def linked_norm_rows(M: int) -> int:
    """Rows that the partial sums of a split norm are kept for in a step of M rows: 16 or 64 in
    a decode step, every row (in whole 64s) otherwise."""
    return lib().picolm_linear_norm_rows(M)


def linked_norm_parts(M: int, N: int, K: int) -> int:
    """Partial sums per row that a product of M rows, N output columns and K input columns leaves
    for the norm that follows: one per workgroup (or column of tiles) of the kernel that finishes
    the rows.  0: that kernel cannot."""
    return lib().picolm_linear_norm_parts(M, N, K)


def gemm_links_norms(a, w, c, epilogue: int, prepares: bool) -> bool:
    """Whether the product for these operands can take part in a norm split between two products:
    prepare the next one (with the accumulating epilogue), or else take a prepared one's
    statistics.  The library decides (picolm_linear_links_norms): it depends on the operands'
    types and on which kernel their sizes get."""
    if a.dim() != 2 or a.dtype not in _DT or w.dtype not in _DT or c.dtype not in _DT:
        return False
    return bool(lib().picolm_linear_links_norms(_ptr(a), dt_of(a), _ptr(w), dt_of(w), dt_of(c), a.shape[0], w.shape[0],
                                                a.shape[1], epilogue, int(prepares)))


def gemm_linked(a, w, c, epilogue: int, prepare=None, prepared=None) -> None:
    """c (=, +=, = silu-gated) a @ w.T through the kernel that the library picks for the operands'
    types and sizes (picolm_linear), optionally next to an RMSNorm that is split between two
    products.

    prepare = (norm weights f32 [N], h_out bf16 [M, N], ssq_out f32 [parts, rows]): with the
    accumulating epilogue, also leave h_out = bf16(c * weights) and the partial sums of c^2.
    prepared = (ssq f32 [parts, rows], row length of the norm, eps): `a` is such an h_out; the
    sums are multiplied by 1 / sqrt(sum(x^2) / length + eps).  rows and parts as
    linked_norm_rows / linked_norm_parts say for the step's M."""
    M, N, K = _gemm_shapes(a, w, c, epilogue)
    rows = linked_norm_rows(M)
    nw = nh = nssq = ssq = None
    next_parts = n_parts = norm_len = 0
    eps = 0.0
    if prepare is not None:
        nw, nh, nssq = prepare
        _dev("gemm_linked.norm_weight", nw, torch.float32, 1)
        _dev("gemm_linked.h_out", nh, torch.bfloat16, 2)
        _dev("gemm_linked.ssq_out", nssq, torch.float32, 2)
        next_parts = nssq.shape[0]
        if nw.numel() != N or tuple(nh.shape) != (M, N) or nssq.shape[1] != rows:
            raise KernelError("gemm_linked: the buffers for the next norm do not fit the product")
    if prepared is not None:
        ssq, norm_len, eps = prepared
        _dev("gemm_linked.ssq", ssq, torch.float32, 2)
        n_parts = ssq.shape[0]
        if ssq.shape[1] != rows:
            raise KernelError("gemm_linked: the statistics are not those of this product's input rows")
    _check(lib().picolm_linear(_ptr(a), dt_of(a), _ptr(w), dt_of(w), _ptr(c), dt_of(c), M, N, K, epilogue,
                               _ptr(nw), _ptr(nh), _ptr(nssq), next_parts, _ptr(ssq), n_parts, int(norm_len), c_float(eps),
                               _ptr(splitk_workspace(a.device)), _stream()))


def gemm(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int = EPI_STORE) -> None:
    """The product the engine calls: the library picks the kernel for the operands' types and sizes."""
    gemm_linked(a, w, c, epilogue)


def attn_mfma_takes(q: torch.Tensor, d: int) -> bool:
    return q.dtype == torch.bfloat16 and bool(lib().picolm_attn_mfma_takes(d))


def attn_prefill_mfma(q, k_pages, v_pages, out, batch, page_table, ring_pages, H, G, d, window, scale) -> None:
    _attn_check(q, k_pages, v_pages, out, page_table, H, G, d)
    tile_seq, tile_q0, n_tiles = batch.prefill_tiles(lib().picolm_attn_prefill_mfma_tile_tokens(H, G))
    _check(lib().picolm_attn_prefill_mfma(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(tile_seq), _ptr(tile_q0), n_tiles,
        _ptr(batch.seq_slot), _ptr(batch.seq_pos0), _ptr(batch.seq_nnew), _ptr(batch.cu_seqlens), _ptr(page_table),
        page_table.shape[1], ring_pages, H, G, d, window, c_float(scale), _stream()))


def kv_store_tiles(qkv, k_pages, v_pages, cos, sin, style: int, batch, page_table, ring_pages: int, H: int, G: int, d: int) -> None:
    """Keys (rotated) and values of a prefill step's tokens into the cache, over the tiles of the
    matrix-core attention kernel; q is left to that kernel (attn_prefill_rope)."""
    _dev("kv_store.qkv", qkv, torch.float32, 2)
    if qkv.shape[1] != (H + 2 * G) * d or qkv.shape[0] < batch.T:
        raise KernelError(f"kv_store_tiles: qkv {tuple(qkv.shape)} is not [{batch.T}, {(H + 2 * G) * d}]")
    _check_pages("kv_store_tiles", k_pages, v_pages, k_pages.dtype, G, d)
    _dev("kv_store.page_table", page_table, torch.int32, 2)
    if cos is not None:
        _dev("kv_store.cos", cos, torch.float32, 2)
        _dev("kv_store.sin", sin, torch.float32, 2)
        if cos.shape[1] != d // 2 or sin.shape != cos.shape or cos.shape[0] < batch.max_len:
            raise KernelError(f"kv_store_tiles: tables {tuple(cos.shape)} do not cover {batch.max_len} positions of d/2 = {d // 2}")
    tile_tokens = lib().picolm_attn_prefill_mfma_tile_tokens(H, G)
    tile_seq, tile_q0, n_tiles = batch.prefill_tiles(tile_tokens)
    _check(lib().picolm_kv_store_tiles(
        _ptr(qkv), _ptr(k_pages), _ptr(v_pages), dt_of(k_pages), _ptr(cos), _ptr(sin), style, _ptr(tile_seq), _ptr(tile_q0),
        n_tiles, tile_tokens, _ptr(batch.seq_slot), _ptr(batch.seq_pos0), _ptr(batch.seq_nnew), _ptr(batch.cu_seqlens),
        _ptr(page_table), page_table.shape[1], ring_pages, H, G, d, _stream()))


def attn_prefill_rope(qkv, k_pages, v_pages, out, batch, page_table, ring_pages, H, G, d, window, scale, cos, sin, style) -> None:
    """attn_prefill_mfma with q taken from the float rows qkv [T, (H+2G)d] and rotated inside the
    kernel (cos, sin None: no rotation).  The step's keys and values must be in the cache already
    (rope_kv_store with q_out None)."""
    _dev("attn.qkv", qkv, torch.float32, 2)
    if qkv.shape[1] != (H + 2 * G) * d or qkv.shape[0] < batch.T:
        raise KernelError(f"attn_prefill_rope: qkv {tuple(qkv.shape)} is not [{batch.T}, {(H + 2 * G) * d}]")
    _dev("attn.out", out, torch.bfloat16, 2)
    if tuple(out.shape) != (qkv.shape[0], H * d):
        raise KernelError(f"attn_prefill_rope: out {tuple(out.shape)} is not {(qkv.shape[0], H * d)}")
    _check_pages("attn_prefill_rope", k_pages, v_pages, torch.bfloat16, G, d)
    _dev("attn.page_table", page_table, torch.int32, 2)
    if cos is not None:
        _dev("attn.cos", cos, torch.float32, 2)
        _dev("attn.sin", sin, torch.float32, 2)
        if cos.shape[1] != d // 2 or sin.shape != cos.shape or cos.shape[0] < batch.max_len:
            raise KernelError(f"attn_prefill_rope: tables {tuple(cos.shape)} do not cover {batch.max_len} positions of d/2 = {d // 2}")
    tile_seq, tile_q0, n_tiles = batch.prefill_tiles(lib().picolm_attn_prefill_mfma_tile_tokens(H, G))
    _check(lib().picolm_attn_prefill_rope_mfma(
        _ptr(qkv), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(tile_seq), _ptr(tile_q0), n_tiles,
        _ptr(batch.seq_slot), _ptr(batch.seq_pos0), _ptr(batch.seq_nnew), _ptr(batch.cu_seqlens), _ptr(page_table),
        page_table.shape[1], ring_pages, H, G, d, window, c_float(scale), _ptr(cos), _ptr(sin), style, _stream()))


def attn_decode_counters(n_seq: int, H: int, G: int) -> int:
    """Counters (int32, zero between launches) with which the matrix-core decode kernels combine
    the chunks of a sequence themselves: one per sequence and workgroup of heads."""
    return n_seq * G * ((H // G + 31) // 32)


def _counters_check(chunks_done, n_seq, H, G):
    if chunks_done is not None:
        _i32("attn.chunks_done", chunks_done, attn_decode_counters(n_seq, H, G))


def attn_decode_mfma(q, k_pages, v_pages, out, partial, n_seq, chunk_list, n_chunks, pages_per_chunk,
                     max_splits, seq_pos0, page_table, ring_pages, H, G, d, window, scale, chunks_done=None) -> None:
    """chunks_done: see attn_decode_counters; None lets a second kernel combine the chunks."""
    _attn_check(q, k_pages, v_pages, out, page_table, H, G, d)
    _decode_check(q, partial, n_seq, chunk_list, n_chunks, pages_per_chunk, max_splits, seq_pos0, H, d)
    _counters_check(chunks_done, n_seq, H, G)
    _check(lib().picolm_attn_decode_mfma(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(partial if max_splits > 1 else None), n_seq,
        _ptr(chunk_list), n_chunks, pages_per_chunk, max_splits, _ptr(seq_pos0), _ptr(page_table),
        page_table.shape[1], ring_pages, H, G, d, window, c_float(scale), _ptr(chunks_done), _stream()))


def attn_decode_rope(qkv, k_pages, v_pages, out, partial, n_seq, chunk_list, n_chunks, pages_per_chunk, max_splits,
                     seq_pos0, page_table, ring_pages, H, G, d, window, scale, cos, sin, style, tok_page,
                     chunks_done=None) -> None:
    """A decode step's rotation, cache write and attention in one launch (bfloat16 cache, head
    sizes of the matrix-core kernels): `qkv` are the float rows [n_seq, (H+2G)d] of the new tokens,
    `tok_page[i]` the physical page that takes sequence i's new key and value.  chunks_done: see
    attn_decode_counters."""
    _counters_check(chunks_done, n_seq, H, G)
    _dev("attn.qkv", qkv, torch.float32, 2)
    if qkv.shape[0] < n_seq or qkv.shape[1] != (H + 2 * G) * d:
        raise KernelError(f"attn_decode_rope: qkv {tuple(qkv.shape)} is not [>= {n_seq}, {(H + 2 * G) * d}]")
    _dev("attn.out", out, torch.bfloat16, 2)
    if out.shape[0] < n_seq or out.shape[1] != H * d:
        raise KernelError(f"attn_decode_rope: out {tuple(out.shape)} is not [>= {n_seq}, {H * d}]")
    _check_pages("attn", k_pages, v_pages, torch.bfloat16, G, d)
    _dev("attn.page_table", page_table, torch.int32, 2)
    if max_splits > 1:
        _dev("attn.partial", partial, torch.float32)
        if partial.numel() < n_seq * H * max_splits * (d + 2):
            raise KernelError("attn_decode_rope: the partial buffer is too small")
    if pages_per_chunk < 1 or max_splits < 1:
        raise KernelError(f"attn_decode_rope: {pages_per_chunk} pages a chunk, {max_splits} chunks a sequence")
    _i32("attn.chunk_list", chunk_list, 8 * (n_chunks + 1))
    _i32("attn.seq_pos0", seq_pos0, n_seq)
    _i32("attn.tok_page", tok_page, n_seq)
    if cos is not None:
        _dev("rope.cos", cos, torch.float32, 2)
        _dev("rope.sin", sin, torch.float32, 2)
        if cos.shape[1] != d // 2 or sin.shape != cos.shape:
            raise KernelError(f"rope: tables {tuple(cos.shape)} do not have d/2 = {d // 2} columns")
    _check(lib().picolm_attn_decode_rope_mfma(
        _ptr(qkv), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(partial if max_splits > 1 else None), n_seq,
        _ptr(chunk_list), n_chunks, pages_per_chunk, max_splits, _ptr(seq_pos0), _ptr(page_table),
        page_table.shape[1], ring_pages, H, G, d, window, c_float(scale), _ptr(cos), _ptr(sin), style, _ptr(tok_page),
        _ptr(chunks_done), _stream()))


def attn_prefill(q, k_pages, v_pages, out, batch, page_table, ring_pages, H, G, d, window, scale) -> None:
    """Attention of a step's new tokens over their sequences' cache pages."""
    if attn_mfma_takes(q, d):
        attn_prefill_mfma(q, k_pages, v_pages, out, batch, page_table, ring_pages, H, G, d, window, scale)
        return
    tile_seq, tile_q0, n_tiles = batch.prefill_tiles(attn_prefill_tile_rows())
    attn_prefill_generic(q, k_pages, v_pages, out, tile_seq, tile_q0, n_tiles, batch.seq_slot, batch.seq_pos0,
                         batch.seq_nnew, batch.cu_seqlens, page_table, ring_pages, H, G, d, window, scale)


def attn_decode(q, k_pages, v_pages, out, partial, n_seq, chunk_list, n_chunks, pages_per_chunk, max_splits,
                seq_pos0, page_table, ring_pages, H, G, d, window, scale, chunks_done=None) -> None:
    """Attention of one new token per sequence (row i of q is sequence i) over its cache pages.
    `chunk_list` is the step's work list, eight ints an entry behind a header entry: entry 1 + x
    gives workgroup x `pages_per_chunk` pages of one sequence.  chunks_done: counters for the
    kernels that can combine a sequence's chunks themselves (attn_decode_counters)."""
    if attn_mfma_takes(q, d):
        attn_decode_mfma(q, k_pages, v_pages, out, partial, n_seq, chunk_list, n_chunks, pages_per_chunk, max_splits,
                         seq_pos0, page_table, ring_pages, H, G, d, window, scale, chunks_done)
    else:
        attn_decode_generic(q, k_pages, v_pages, out, partial, n_seq, chunk_list, n_chunks, pages_per_chunk,
                            max_splits, seq_pos0, page_table, ring_pages, H, G, d, window, scale)


def sample_scratch_bytes(n_rows: int, V: int, temperature: float, top_k: int) -> int:
    """Scratch memory with which `sample` spreads a row over many workgroups (0: it cannot)."""
    return lib().picolm_sample_scratch_bytes(n_rows, V, c_float(temperature), int(top_k))


def sample(logits: torch.Tensor, out: torch.Tensor, temperature: float, top_k: int, top_p: float,
           min_p: float, rng_states: torch.Tensor | None, state_index: torch.Tensor | None,
           scratch: torch.Tensor | None = None) -> None:
    """One token per row of `logits`; `rng_states` (int64 bits of xorshift64 states) advance.
    `scratch` (uint8, sample_scratch_bytes): without it one workgroup per row does all the work."""
    _dev("sample.logits", logits, torch.float32, 2)
    n, V = logits.shape
    _i32("sample.out", out, n)
    if temperature > 0:
        _dev("sample.rng_states", rng_states, torch.int64, 1)
        if state_index is not None:
            _i32("sample.state_index", state_index, n)
        elif rng_states.numel() < n:
            raise KernelError("sample: fewer generator states than rows")
    if scratch is not None:
        _dev("sample.scratch", scratch, torch.uint8)
    _check(lib().picolm_sample(_ptr(logits), c_int64(V), n, V, c_float(temperature), int(top_k), c_float(top_p),
                               c_float(min_p), _ptr(rng_states), _ptr(state_index), _ptr(out), _ptr(scratch),
                               c_int64(scratch.numel() if scratch is not None else 0), _stream()))


def read_probe(src: torch.Tensor, sink: torch.Tensor, blocks: int = 2048, streaming: bool = True) -> int:
    """Queue one sweep over `src` (each workgroup a contiguous share; non-temporal loads if
    `streaming`, as the kernels load what a launch reads once); returns the bytes it reads."""
    _dev("read_probe.src", src)
    _dev("read_probe.sink", sink, torch.int32)
    nbytes = src.numel() * src.element_size()
    nbytes -= nbytes % 16
    _check(lib().picolm_read_probe(_ptr(src), ctypes.c_size_t(nbytes), _ptr(sink), blocks, int(streaming), _stream()))
    return int(lib().picolm_read_probe_bytes(ctypes.c_size_t(nbytes), blocks))


def mfma_probe(sink: torch.Tensor, blocks: int, iters: int, random_operands: bool = False) -> float:
    """Queue a compute-only MFMA kernel (on small integers, or on pseudo-random values that make
    the GPU draw the power real data does); returns the flops it performs."""
    _dev("mfma_probe.sink", sink, torch.float32)
    _check(lib().picolm_mfma_probe(_ptr(sink), blocks, iters, int(random_operands), _stream()))
    return blocks * 4 * iters * 8 * 32768.0
