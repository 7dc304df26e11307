#!/usr/bin/env python3
"""Decode and prefill throughput of the Llama-3.1-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]

A step is one decode step of the generation loop's inner body: the model step over the
batch from the cache, the sampler, and the hand-over of the sampled tokens.  Weights are
random bf16 N(0, 0.02) made on the GPU, prompts are seeded uniform-random token ids with
lengths uniform in [128, 2048]; context is capped at 4096.  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

LLAMA31_8B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
    num_key_value_heads=8, num_hidden_layers=32, vocab_size=128256, head_dim=128, rms_norm_eps=1e-5,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=False, max_position_embeddings=131072, eos_token_id=128001, bos_token_id=128000)
CONTEXT = 4096
PREFILL_TOKENS = 2048


def weight_bytes(cfg, itemsize=2) -> int:
    D, F, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    per_layer = D * (cfg.q_size + 2 * cfg.kv_size) + cfg.q_size * D + 3 * D * F
    return (L * per_layer + V * D) * itemsize + (L * 2 * D + D) * 4


def kv_bytes_per_token(cfg, itemsize=2) -> int:
    return 2 * cfg.num_hidden_layers * cfg.kv_size * itemsize


def prefill_flops(cfg, T: int) -> float:
    D, F, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    gemm = 2.0 * T * (D * (cfg.q_size + 2 * cfg.kv_size) + cfg.q_size * D + 3 * D * F)
    attn = 4.0 * cfg.head_dim * cfg.num_attention_heads * (T * (T + 1) / 2)
    return L * (gemm + attn) + 2.0 * D * V


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the 32 of the shape (0: all)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--prefill-only", action="store_true", help="run only the 2,048-token prefill (for profiling)")
    ap.add_argument("--batch-only", action="store_true", help="run only the decode at --batch (for profiling)")
    ap.add_argument("--sampling", choices=["greedy", "picolm"], default="greedy",
                    help="greedy (the measured default) or picolm's command-line defaults: temperature 0.8, top_k 40, top_p 0.9, min_p 0.05")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="with --prefill-only: a prompt of another length than the 2,048 of the record")
    ap.add_argument("--prompt-range", default="128,2048",
                    help="prompt lengths of the decode runs, uniform in LO,HI (the record's are 128,2048)")
    ap.add_argument("--context", type=int, default=CONTEXT, help="longest sequence the cache is laid out for")
    ap.add_argument("--steps-ahead", type=int, choices=[0, 1], default=1,
                    help="1 (the generation loop's way): the next step is launched before this step's tokens are "
                         "read on the host; 0: the host reads every step's tokens first")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU library")
        return 2

    import torch

    from picolm_amd import LlamaConfig
    from picolm_amd.engine import Session, random_model
    from picolm_amd.sampling import Sampler, SamplingParams
    from picolm_amd.sampling.params import CLI_DEFAULTS

    full_layers = LLAMA31_8B["num_hidden_layers"]
    cfg_dict = dict(LLAMA31_8B)
    if args.layers:
        cfg_dict["num_hidden_layers"] = args.layers
    cfg = LlamaConfig.from_dict(cfg_dict)
    dev = torch.device("cuda:0")
    t0 = time.time()
    model = random_model(cfg, seed=0, std=0.02, dtype="bfloat16", device=dev)
    torch.cuda.synchronize()
    print(f"[bench] model of {cfg.num_hidden_layers} layers ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    prompt_lo, prompt_hi = (int(x) for x in args.prompt_range.split(","))
    context = args.context

    def decode_run(batch: int, steps: int, warmup: int):
        lens = [int(x) for x in rng.integers(prompt_lo, prompt_hi + 1, size=batch)]
        prompts = [[int(t) for t in rng.integers(0, cfg.vocab_size, size=n)] for n in lens]
        pages = sum((min(n + steps + warmup + 1, context) + 63) // 64 for n in lens)
        sess = Session(model, max_tokens=pages * 64, max_seq_len=context, n_slots=batch)
        sampler = Sampler(CLI_DEFAULTS if args.sampling == "picolm" else SamplingParams(), batch, dev)
        slots = sess.begin(batch)
        # prompts go in one at a time here only to bound the workspace of this harness
        rows = []
        for s, p in zip(slots, prompts):
            rows.append(sess.step([s], [p]).clone())
        logits = torch.cat(rows)
        idx = list(range(batch))

        if args.steps_ahead:
            # as the generation loop runs: a step takes its tokens on the device from the draw
            # before it, and the host reads a step's tokens while the next step runs
            def one_step(pending):
                lg = sess.step_tokens_on_device(slots, pending.on_device())
                nxt = sampler.launch(lg, idx)
                pending.wait()
                return nxt

            state = sampler.launch(logits, idx)
        else:
            def one_step(lg):
                toks = sampler.sample(lg, idx)
                return sess.step(slots, [[t] for t in toks])

            state = logits
        for _ in range(warmup):
            state = one_step(state)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            state = one_step(state)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx = sum(sess.length(s) for s in slots) - batch * steps / 2.0     # mean live context over the timed steps
        sess.release(slots)
        del sess
        torch.cuda.empty_cache()
        return batch * steps / dt, dt / steps, ctx

    def prefill_run(T: int, reps: int = 3):
        sess = Session(model, max_tokens=T + 64, max_seq_len=max(context, T + 64), n_slots=1)
        toks = [int(t) for t in rng.integers(0, cfg.vocab_size, size=T)]
        times = []
        for _ in range(reps + 1):
            [s] = sess.begin(1)
            torch.cuda.synchronize()
            t = time.perf_counter()
            sess.step([s], [toks])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            sess.release([s])
        del sess
        torch.cuda.empty_cache()
        return float(np.median(times[1:]))

    if args.prefill_only:
        sec = prefill_run(args.prefill_tokens)
        print(json.dumps({"prefill_ms": round(sec * 1e3, 3), "tokens": args.prefill_tokens, "layers": cfg.num_hidden_layers}))
        return 0
    tok_s, s_per_step, ctx_tokens = decode_run(args.batch, args.steps, args.warmup)
    step_bytes = weight_bytes(cfg) + ctx_tokens * kv_bytes_per_token(cfg)
    achieved = step_bytes / s_per_step / 1e9
    record = {
        "metric": "decode tok/s at batch 8 (Llama-3.1-8B shape, bf16, context <= 4096)",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(s_per_step * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": f"synthetic: random bf16 weights N(0,0.02), seeded uniform-random token ids, prompt lengths uniform in [{prompt_lo},{prompt_hi}]",
        "config": {
            "model": "Llama-3.1-8B shape", "layers": cfg.num_hidden_layers, "layers_of_shape": full_layers,
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "rope_theta": cfg.rope_theta, "rope_scaling": "llama3 factor 8 low 1 high 4 original 8192",
            "rms_norm_eps": cfg.rms_norm_eps, "tied": cfg.tie_word_embeddings, "global_batch": args.batch,
            "seq_len": context, "prompt_lengths": f"uniform[{prompt_lo},{prompt_hi}]", "mean_context": round(ctx_tokens / args.batch, 1),
            "sampling": args.sampling, "steps_ahead": args.steps_ahead, "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not (args.no_points or args.batch_only):
        sec = prefill_run(PREFILL_TOKENS)
        fl = prefill_flops(cfg, PREFILL_TOKENS)
        record["prefill"] = {"value": round(PREFILL_TOKENS / sec, 1), "tokens": PREFILL_TOKENS, "ms": round(sec * 1e3, 3),
                             "frac": round(fl / sec / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
        b1, _, _ = decode_run(1, min(args.steps, 32), min(args.warmup, 4))
        b64, _, _ = decode_run(64, min(args.steps, 16), min(args.warmup, 2))
        record["points"] = {"decode_b1": round(b1, 2), "decode_b64": round(b64, 2)}
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
