"""Drives ``bin/trace_run`` as a user would: a child process fed one JSON step per line, each step
acknowledged by ``done <step>``; logits are read from the files it writes."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
TRACE_RUN = ROOT / "bin" / "trace_run"


class Replay:
    def __init__(self, model_dir, dtype: str, out_dir, max_tokens: int, extra=()):
        self.out = Path(out_dir)
        self.out.mkdir(parents=True, exist_ok=True)
        self.proc = subprocess.Popen(
            [sys.executable, str(TRACE_RUN), "--model", str(model_dir), "--dtype", dtype, "--out", str(self.out),
             "--max-tokens", str(max_tokens), *extra],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1,
        )
        self.vocab = json.loads((Path(model_dir) / "config.json").read_text())["vocab_size"]
        self.step_no = 0

    def step(self, entries, end=()):
        """``entries``: list of (id, tokens, want). Returns float32 ``[wanted, vocab]`` or None."""
        n = self.step_no
        self.step_no += 1
        msg = {"step": n, "entries": [{"id": i, "tokens": list(map(int, t)), "want": list(map(int, w))} for i, t, w in entries],
               "end": list(end)}
        self.proc.stdin.write(json.dumps(msg) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline()
        if line.strip() != f"done {n}":
            rest = self.proc.stdout.read()
            raise RuntimeError(f"trace_run answered {line!r} to step {n} (exit {self.proc.poll()}): {rest[-2000:]}")
        wanted = sum(len(w) for _, _, w in entries)
        f = self.out / f"{n}.f32"
        if wanted == 0:
            assert not f.exists()
            return None
        return np.fromfile(f, dtype="<f4").reshape(wanted, self.vocab)

    def close(self) -> int:
        self.proc.stdin.close()
        rc = self.proc.wait(timeout=120)
        return rc

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        if self.proc.poll() is None:
            try:
                self.proc.stdin.close()
            except OSError:
                pass
            try:
                self.proc.wait(timeout=60)
            except subprocess.TimeoutExpired:
                self.proc.kill()
        return False


def round64(n: int) -> int:
    return -(-n // 64) * 64
