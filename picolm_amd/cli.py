"""Command line in picolm's manner (picolm/picolm.c:140-196, :820-940): a model, a prompt from
-p or standard input, -n, -t, -k, --top-p, -s, -c.  Tokenizers are outside this library, so
the prompt is token ids (integers separated by blanks or commas) and the output is the
generated ids, one line per prompt; each line of standard input or of --batch-file is one
prompt, and several lines make a batch.  Timings go to standard error in picolm's format
(picolm/picolm.c:1628-1636).

  picolm <model_dir> [-p "1 5 17"] [-n 256] [-t 0.8] [-k 40] [--top-p 0.9] [--min-p 0.05]
         [-s 42] [-c CONTEXT] [--dtype bfloat16|float32] [--batch-file FILE] [--batch N]
  picolm --random-model OUT_DIR --config CONFIG.json [-s SEED] [--std 0.02] [--norm-sigma 0]
  picolm <model_dir> --benchmark [-p ...] [-n N]         prompt and generation again and again
  picolm <model_dir> --benchmark-ctx [-p ...] [-n N] [-c CONTEXT]     speed over a growing context (CSV)
  picolm --gpu-diff S I O | --gpu-attn-diff N_TOK N_HEADS N_KV_HEADS HEAD_DIM     kernels against slow ones
  picolm <model_dir> --list-tensors | --list-kv
"""
from __future__ import annotations

import argparse
import json
import re
import sys

from .sampling.params import CLI_DEFAULTS, SamplingParams


def parse_ids(text: str) -> list[int]:
    toks = [t for t in re.split(r"[\s,]+", text.strip()) if t]
    try:
        return [int(t) for t in toks]
    except ValueError as e:
        raise SystemExit(f"the prompt must be token ids (integers): {e}") from None


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="picolm", description="Llama text generation on MI355X: token ids in, token ids out")
    ap.add_argument("model", nargs="?", help="folder with config.json and model.safetensors")
    ap.add_argument("-p", dest="prompt", help="prompt as token ids (else standard input)")
    ap.add_argument("-n", dest="max_tokens", type=int, default=256, help="max tokens to generate (default 256)")
    ap.add_argument("-t", dest="temperature", type=float, default=CLI_DEFAULTS.temperature,
                    help="temperature (default 0.8, 0 = greedy)")
    ap.add_argument("-k", dest="top_k", type=int, default=CLI_DEFAULTS.top_k, help="top-k (default 40, 0 = off)")
    ap.add_argument("--top-p", dest="top_p", type=float, default=CLI_DEFAULTS.top_p, help="nucleus (default 0.9)")
    ap.add_argument("--min-p", dest="min_p", type=float, default=CLI_DEFAULTS.min_p, help="min-p (default 0.05)")
    ap.add_argument("-s", dest="seed", type=int, default=CLI_DEFAULTS.seed, help="RNG seed (default 42)")
    ap.add_argument("-c", dest="context", type=int, default=0, help="context length override")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch-file", help="file with one prompt of token ids per line")
    ap.add_argument("--batch", type=int, default=64, help="most sequences in one batch (default 64)")
    ap.add_argument("--json", action="store_true", help="print one JSON record with tokens and timings")
    ap.add_argument("--random-model", metavar="OUT_DIR", help="write a model folder with random weights and exit")
    ap.add_argument("--config", help="config.json for --random-model")
    ap.add_argument("--std", type=float, default=0.02)
    ap.add_argument("--norm-sigma", type=float, default=0.0)
    ap.add_argument("--list-tensors", action="store_true", help="list the model folder's tensors and exit")
    ap.add_argument("--list-kv", action="store_true", help="list the model folder's metadata entries and exit")
    ap.add_argument("--gpu-diff", nargs=3, type=int, metavar=("S", "I", "O"),
                    help="diff the product kernels (matrix cores, 32-bit, float64 on the host) on random input: S rows, I inputs, O outputs")
    ap.add_argument("--gpu-attn-diff", nargs=4, type=int, metavar=("N_TOK", "N_HEADS", "N_KV_HEADS", "HEAD_DIM"),
                    help="diff the attention kernels (bfloat16, 32-bit, float64 on the host) on random q, k, v")
    ap.add_argument("--benchmark-ctx", action="store_true",
                    help="prefill and generation speed at growing context sizes: -p is appended and answered over the cached "
                         "context, then -n tokens are generated, until -c is full; CSV ctx_size,prefill_tok/s,gen_tok/s")
    ap.add_argument("--benchmark", action="store_true", help="continuous benchmark loop (Ctrl-C to stop)")
    ap.add_argument("--benchmark-iterations", type=int, default=0, help="stop --benchmark after this many rounds (0: never)")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.random_model:
        from .config import read_config_json, resolve
        from .weights import write_random_model
        if not args.config:
            raise SystemExit("--random-model needs --config CONFIG.json")
        d = read_config_json(args.config)
        cfg = resolve(d).parse_config(d)
        write_random_model(cfg, args.random_model, seed=args.seed, std=args.std, norm_sigma=args.norm_sigma)
        print(args.random_model)
        return 0
    if args.gpu_diff:              # stand-alone kernel checks: no model needed (picolm.c:950-963)
        from .diagnostics import gpu_diff
        return gpu_diff(*args.gpu_diff, seed=args.seed)
    if args.gpu_attn_diff:
        from .diagnostics import gpu_attn_diff
        return gpu_attn_diff(*args.gpu_attn_diff, seed=args.seed)
    if not args.model:
        build_parser().print_usage(sys.stderr)
        print("No model folder specified", file=sys.stderr)
        return 1
    if args.list_tensors:
        from .weights import Checkpoint
        ck = Checkpoint(args.model)
        for n in sorted(ck.names()):
            dt, shape = ck.info(n)
            print(f"{n}\t{list(shape)}\t{str(dt).replace('torch.', '')}")
        return 0
    if args.list_kv:
        from .diagnostics import list_kv
        return list_kv(args.model)
    if args.batch_file:
        with open(args.batch_file) as f:
            lines = [l for l in f.read().splitlines() if l.strip()]
    elif args.prompt is not None:
        lines = [args.prompt]
    elif not sys.stdin.isatty():
        lines = [l for l in sys.stdin.read().splitlines() if l.strip()]
    else:
        lines = []
    prompts = [parse_ids(l) for l in lines]

    from .cache import PAGE_TOKENS, pages_for
    from .engine import Session, load_model
    from .generation import generate
    model = load_model(args.model, dtype=args.dtype)
    cfg = model.config
    if not prompts:
        # picolm starts from BOS without a prompt (picolm.c:1532-1535); an architecture whose
        # configuration names no start token needs a prompt
        bos = getattr(cfg, "bos_token_id", None)
        if bos is None:
            raise SystemExit("no prompt given, and this model's configuration names no start token (bos_token_id)")
        prompts = [[int(bos)]]
    context = args.context or cfg.max_position_embeddings
    params = SamplingParams(args.temperature, args.top_k, args.top_p, args.min_p, args.seed)
    if args.benchmark or args.benchmark_ctx:        # one sequence, speed only (picolm.c:969-976, :1311)
        from . import diagnostics
        context = min(context, cfg.max_position_embeddings)
        session = Session(model, max_tokens=pages_for(context) * PAGE_TOKENS, max_seq_len=context, n_slots=1)
        if args.benchmark_ctx:
            return diagnostics.benchmark_ctx(session, prompts[0], args.max_tokens, context, params)
        return diagnostics.benchmark(session, prompts[0], args.max_tokens, params, args.benchmark_iterations)
    per = sorted((pages_for(min(len(p) + args.max_tokens, context)) for p in prompts), reverse=True)
    session = Session(model, max_tokens=max(1, sum(per[:args.batch])) * PAGE_TOKENS, max_seq_len=context)
    results, stats = generate(session, prompts, args.max_tokens, params, batch_size=args.batch, return_stats=True)
    if args.json:
        print(json.dumps({"tokens": [r.tokens for r in results], "finish": [r.finish for r in results],
                          "prefill_tokens": stats.prompt_tokens, "prefill_seconds": stats.prefill_seconds,
                          "generated_tokens": stats.generated_tokens, "decode_seconds": stats.decode_seconds}))
    else:
        for r in results:
            print(" ".join(str(t) for t in r.tokens))
    sys.stdout.flush()
    pre, gen = stats.prefill_seconds, stats.decode_seconds
    print("---", file=sys.stderr)
    print(f"Prefill: {stats.prompt_tokens} tokens in {pre:.2f}s ({stats.prompt_tokens / pre if pre > 0 else 0:.1f} tok/s)",
          file=sys.stderr)
    print(f"Generation: {stats.generated_tokens} tokens in {gen:.2f}s "
          f"({stats.generated_tokens / gen if gen > 0 else 0:.1f} tok/s)", file=sys.stderr)
    print(f"Total: {pre + gen:.2f}s", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
