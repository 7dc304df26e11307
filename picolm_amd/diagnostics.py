"""The command line's self-checks and speed runs, in picolm's manner and with its option names:
--gpu-diff and --gpu-attn-diff compare the fast kernels with slow ones on random input
(picolm/picolm.c:162-168, :895-905, :950-963), --benchmark-ctx measures prefill and generation
speed over a growing cached context (picolm/picolm.c:405-547), --benchmark repeats prompt and
generation until interrupted (picolm/picolm.c:1311-1470, summary :358-385), --list-kv lists the
model's metadata (picolm/picolm.c:187).  picolm compares its tensor-core kernels with its scalar
GPU kernels; here the matrix-core bfloat16 kernels are compared with the 32-bit kernels of the same
library and both with float64 arithmetic on the host.
"""
from __future__ import annotations

import json
import math
import os
import sys
import time

import torch


def _say(*a) -> None:
    print(*a, file=sys.stderr, flush=True)


def _device() -> torch.device:
    if not torch.cuda.is_available():
        raise SystemExit("no GPU: this check runs the library's kernels")
    return torch.device("cuda:0")


def _diff_line(name: str, got: torch.Tensor, ref: torch.Tensor) -> float:
    err = (got.double().cpu() - ref).abs()
    scale = max(1.0, float(ref.abs().max()))
    worst = int(err.argmax())
    _say(f"  {name}: max abs diff {float(err.max()):.3e} (of values up to {scale:.3f}) at element {worst}, "
         f"mean abs diff {float(err.mean()):.3e}")
    return float(err.max()) / scale


def gpu_diff(S: int, I: int, O: int, seed: int = 42) -> int:
    """C[S, O] = A[S, I] W[O, I]^T on random operands: the matrix-core product as the engine picks
    it for S rows, the 32-bit product of the same (bfloat16-valued) operands, float64 on the host."""
    from . import kernels
    if min(S, I, O) < 1:
        raise SystemExit("--gpu-diff S I O: three positive sizes")
    dev = _device()
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(S, I, generator=g).to(torch.bfloat16)
    w = (torch.randn(O, I, generator=g) / math.sqrt(I)).to(torch.bfloat16)
    ref = a.double() @ w.double().T
    _say(f"GPU product diff: {S} rows, {I} inputs, {O} outputs, seed {seed}")
    c16 = torch.zeros(S, O, dtype=torch.float32, device=dev)
    kernels.gemm(a.to(dev), w.to(dev), c16, kernels.EPI_STORE)
    c32 = torch.zeros(S, O, dtype=torch.float32, device=dev)
    kernels.gemm(a.float().to(dev), w.float().to(dev), c32, kernels.EPI_STORE)
    torch.cuda.synchronize()
    e32 = _diff_line("32-bit kernel against float64", c32, ref)
    e16 = _diff_line("matrix-core kernel against float64", c16, ref)
    _diff_line("matrix-core kernel against 32-bit kernel", c16, c32.double().cpu())
    ok = e32 <= 1e-5 * math.sqrt(I) and e16 <= 1e-5 * math.sqrt(I)      # both sum exact products in float
    _say("PASS" if ok else "FAIL")
    return 0 if ok else 1


class _OneSequence:
    """The index arrays of a step that brings one sequence's first n tokens, as the attention
    kernels read them (the engine plans such arrays for every step)."""

    def __init__(self, n: int, dev):
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
        self.n_seq, self.T, self.max_len = 1, n, n
        self.seq_slot, self.seq_pos0, self.seq_nnew, self.cu_seqlens = i32([0]), i32([0]), i32([n]), i32([0, n])
        self.tok_pos = torch.arange(n, dtype=torch.int32, device=dev)
        self._dev = dev

    def prefill_tiles(self, rows_per_tile: int):
        q0 = list(range(0, self.T, rows_per_tile))          # in the order of the keys they see
        return (torch.zeros(len(q0), dtype=torch.int32, device=self._dev), torch.tensor(q0, dtype=torch.int32, device=self._dev),
                len(q0))


def gpu_attn_diff(n_tok: int, H: int, G: int, d: int, seed: int = 42) -> int:
    """Causal attention of one sequence of n_tok new tokens over a fresh cache: the bfloat16 kernels
    (matrix cores where the head size allows) and the 32-bit kernels, against float64 on the host."""
    from . import kernels
    from .cache import PAGE_TOKENS
    from .parts.attention import MAX_HEAD_DIM
    if min(n_tok, H, G, d) < 1 or H % G or d % 2 or d > MAX_HEAD_DIM:
        raise SystemExit(f"--gpu-attn-diff n_tok n_heads n_kv_heads head_dim: heads in whole groups, an even head size up to {MAX_HEAD_DIM}")
    dev = _device()
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(n_tok, (H + 2 * G) * d, generator=g)
    n_pages = (n_tok + PAGE_TOKENS - 1) // PAGE_TOKENS
    table = torch.arange(n_pages, dtype=torch.int32).reshape(1, n_pages).to(dev)
    scale = 1.0 / math.sqrt(d)
    _say(f"GPU attention diff: {n_tok} tokens, {H} heads on {G} groups of size {d}, seed {seed}")
    outs = {}
    for dtype in (torch.float32, torch.bfloat16):
        batch = _OneSequence(n_tok, dev)
        kp = torch.zeros(n_pages, G, PAGE_TOKENS, d, dtype=dtype, device=dev)
        vp = torch.zeros(n_pages, G, d, PAGE_TOKENS, dtype=dtype, device=dev)
        q = torch.zeros(n_tok, H * d, dtype=dtype, device=dev)
        out = torch.zeros(n_tok, H * d, dtype=dtype, device=dev)
        tok_page = (batch.tok_pos // PAGE_TOKENS).to(torch.int32)
        kernels.rope_kv_store(qkv.to(dev), q, kp, vp, None, None, 0, batch.tok_pos, tok_page, H, G, d)
        kernels.attn_prefill(q, kp, vp, out, batch, table, n_pages, H, G, d, 0, scale)
        outs[dtype] = out
    torch.cuda.synchronize()
    errs = {}
    for dtype, name in ((torch.float32, "32-bit kernels"), (torch.bfloat16, "bfloat16 kernels")):
        # the reference sees what the kernels see: operands rounded to the cache's type
        x = qkv.to(dtype).double().reshape(n_tok, H + 2 * G, d)
        qh, kh, vh = x[:, :H], x[:, H:H + G], x[:, H + G:]
        kh, vh = kh.repeat_interleave(H // G, dim=1), vh.repeat_interleave(H // G, dim=1)
        s = torch.einsum("qhd,khd->hqk", qh, kh) * scale
        s = s.masked_fill(torch.triu(torch.ones(n_tok, n_tok, dtype=torch.bool), 1), float("-inf"))
        ref = torch.einsum("hqk,khd->qhd", torch.softmax(s, dim=-1), vh).reshape(n_tok, H * d)
        errs[dtype] = _diff_line(f"{name} against float64", outs[dtype], ref)
    _diff_line("bfloat16 kernels against 32-bit kernels", outs[torch.bfloat16], outs[torch.float32].double().cpu())
    ok = errs[torch.float32] <= 2e-5 and errs[torch.bfloat16] <= 2e-2
    _say("PASS" if ok else "FAIL")
    return 0 if ok else 1


def list_kv(model_dir: str) -> int:
    """The model folder's metadata: config.json's entries, then what the safetensors headers carry."""
    from .weights import Checkpoint
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    for k in sorted(cfg):
        print(f"config.{k} = {json.dumps(cfg[k])}")
    for k, v in sorted(Checkpoint(model_dir).metadata().items()):
        print(f"safetensors.{k} = {v}")
    return 0


class _Loop:
    """What both speed runs share: a session, one slot at a time, a sampler."""

    def __init__(self, session, params):
        from .sampling import Sampler
        self.s = session
        self.sampler = Sampler(params, 1, session.model.runtime.device)

    def prefill(self, slot: int, tokens) -> tuple[torch.Tensor, float]:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = self.s.step([slot], [tokens])
        torch.cuda.synchronize()
        return logits, time.perf_counter() - t0

    def generate(self, slot: int, logits: torch.Tensor, n: int) -> tuple[torch.Tensor, int, float]:
        """n tokens whatever they are (a speed run does not stop at an end token)."""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = 0
        for _ in range(n):
            tok = self.sampler.sample(logits, [0])[0]
            logits = self.s.step([slot], [[tok]])
            done += 1
        torch.cuda.synchronize()
        return logits, done, time.perf_counter() - t0


def benchmark_ctx(session, base_prompt, tokens_per_step: int, context: int, params) -> int:
    """ctx_size,prefill_tok/s,gen_tok/s as CSV on standard error: at each step the base prompt is
    appended to what the cache holds and answered in one step over the whole cached context, then
    tokens_per_step tokens are generated; until the context is full."""
    if tokens_per_step < 1:
        raise SystemExit("--benchmark-ctx: -n must be at least 1")
    loop = _Loop(session, params)
    (slot,) = session.begin(1)
    _say(f"Base prompt: {len(base_prompt)} tokens")
    _say("ctx_size,prefill_tok/s,gen_tok/s")
    held = 0
    try:
        while held + len(base_prompt) + tokens_per_step <= context:
            logits, t_pre = loop.prefill(slot, base_prompt)
            logits, n_gen, t_gen = loop.generate(slot, logits, tokens_per_step)
            _say(f"{held},{len(base_prompt) / t_pre if t_pre > 0 else 0:.1f},{n_gen / t_gen if t_gen > 0 else 0:.1f}")
            held += len(base_prompt) + n_gen
    finally:
        session.release([slot])
    return 0


def benchmark(session, prompt, max_tokens: int, params, iterations: int = 0) -> int:
    """Prompt and generation again and again from an empty cache, a summary after each round, until
    interrupted (or `iterations` rounds)."""
    loop = _Loop(session, params)
    model = session.model
    n_layers = len(model.order)
    _say("\nBenchmark mode (Ctrl-C to stop)")
    _say(f"  Model: {model.weight_bytes() / 2 ** 30:.1f} GB | GPU: {torch.cuda.get_device_name(0)} | dtype: {model.runtime.dtype}")
    _say(f"  Context: {session.cache.max_seq_len} | KV cache: {session.cache.bytes() / 2 ** 20:.0f} MB")
    _say(f"  Prompt: {len(prompt)} tokens | Generate: {max_tokens} tokens\n")
    it = 0
    try:
        while iterations <= 0 or it < iterations:
            it += 1
            t0 = time.perf_counter()
            (slot,) = session.begin(1)
            try:
                logits, t_pre = loop.prefill(slot, prompt)
                room = session.cache.max_seq_len - len(prompt)
                _, n_gen, t_gen = loop.generate(slot, logits, max(0, min(max_tokens, room)))
            finally:
                session.release([slot])
            _say(f"\n--- Iteration {it} ({time.perf_counter() - t0:.2f}s wall) ---")
            _say(f"  Prefill: {len(prompt)} tokens, {n_layers} layers, {t_pre * 1e3:.1f}ms "
                 f"({len(prompt) / t_pre if t_pre > 0 else 0:.1f} tok/s, {t_pre * 1e3 / n_layers:.2f}ms/layer)")
            if n_gen:
                _say(f"  Generation: {n_gen} tokens, {n_layers} layers, {t_gen * 1e3:.1f}ms "
                     f"({n_gen / t_gen if t_gen > 0 else 0:.1f} tok/s, {t_gen * 1e3 / n_gen:.2f}ms/token, "
                     f"{model.weight_bytes() * n_gen / t_gen / 1e9 if t_gen > 0 else 0:.0f} GB/s of weights)")
            _say(f"  Total wall time: {time.perf_counter() - t0:.2f}s")
            _say("----------------------------------\n")
    except KeyboardInterrupt:
        _say("interrupted")
    return 0
