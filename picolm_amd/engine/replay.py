"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and has no forward pass of its own: every step goes through
`Session.step`, the same function, cache and kernels that generation uses.

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step with wanted rows, `<out>/<step>.f32` holds float32 logits [wanted, vocab] in the
order of the entries and of `want`.  After each step a line `done <step>` is printed.
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np

from .builder import load_model
from .session import Session


class TraceError(ValueError):
    pass


class Replayer:
    def __init__(self, session: Session, out_dir: str):
        self.session = session
        self.out_dir = out_dir
        self.slot_of: dict[str, int] = {}
        os.makedirs(out_dir, exist_ok=True)

    def run_step(self, record: dict) -> None:
        step = record.get("step")
        entries = record.get("entries", [])
        slots, tokens, want = [], [], []
        fresh = []
        try:
            for e in entries:
                rid = str(e["id"])
                toks = [int(t) for t in e["tokens"]]
                if not toks:
                    raise TraceError(f"step {step}: request '{rid}' brings no tokens")
                if rid not in self.slot_of:
                    [s] = self.session.begin(1)
                    self.slot_of[rid] = s
                    fresh.append(rid)
                slots.append(self.slot_of[rid])
                tokens.append(toks)
                want.append([int(w) for w in e.get("want", [])])
            if entries:
                logits = self.session.step(slots, tokens, want)
                if logits.shape[0] > 0:
                    arr = logits.detach().cpu().numpy().astype("<f4", copy=False)
                    tmp = os.path.join(self.out_dir, f".{step}.f32.tmp")
                    arr.tofile(tmp)
                    os.replace(tmp, os.path.join(self.out_dir, f"{step}.f32"))
        except Exception:
            for rid in fresh:           # a failed step leaves no half-started request behind
                self.session.release([self.slot_of.pop(rid)])
            raise
        for rid in record.get("end", []):
            rid = str(rid)
            if rid not in self.slot_of:
                raise TraceError(f"step {step}: request '{rid}' ends but never started")
            self.session.release([self.slot_of.pop(rid)])


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold together, each rounded up to 64")
    args = ap.parse_args(argv)
    model = load_model(args.model, dtype=args.dtype)
    session = Session(model, max_tokens=args.max_tokens)
    rp = Replayer(session, args.out)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        rp.run_step(record)
        sys.stdout.write(f"done {record.get('step')}\n")
        sys.stdout.flush()
    return 0
