"""Drives bin/trace_run as a user would: a subprocess, steps on its standard input, one at a
time, each sent after the previous one's `done` line."""
from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class TraceRun:
    def __init__(self, model_dir, dtype, out_dir, max_tokens, env=None):
        self.out_dir = out_dir
        self.proc = subprocess.Popen(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
             "--out", out_dir, "--max-tokens", str(max_tokens)],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1, env=env)
        self.n = 0

    def step(self, entries, end=()):
        """entries: list of (id, tokens, want); returns float32 logits [wanted, vocab] or None."""
        rec = {"step": self.n, "entries": [{"id": i, "tokens": list(map(int, t)), "want": list(map(int, w))}
                                           for i, t, w in entries], "end": list(end)}
        self.proc.stdin.write(json.dumps(rec) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline()
        if line.strip() != f"done {self.n}":
            rest = self.proc.stdout.read()
            raise RuntimeError(f"trace_run answered {line!r} {rest!r} (exit {self.proc.poll()})")
        path = os.path.join(self.out_dir, f"{self.n}.f32")
        self.n += 1
        n_want = sum(len(w) for _, _, w in entries)
        if n_want == 0:
            assert not os.path.exists(path)
            return None
        arr = np.fromfile(path, dtype="<f4")
        return arr.reshape(n_want, -1)

    def close(self):
        self.proc.stdin.close()
        rc = self.proc.wait(timeout=60)
        assert rc == 0, f"trace_run exited with {rc}"
