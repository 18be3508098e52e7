"""Driving an engine to completion while keeping the time of decode-only steps apart from the time of
steps that carry portions of prompts (the reference's offline harness does the same,
bench/offline.py:210-255): a mean over both says nothing about either."""

from __future__ import annotations

import statistics
import time

from .markers import mark


def run_to_completion(engine, max_steps: int | None = None) -> dict:
    """``engine.step()`` until nothing is unfinished. The wall time of a call is booked to the kind of
    the batch it returns: the one whose tokens it waited for (with the read-back one step behind the
    launch that is the previous launch, whose device time the call spent waiting)."""
    from ..engine.scheduler import Phase

    times = {Phase.DECODE: [], Phase.MIXED: [], Phase.PREFILL: []}
    rows = {Phase.DECODE: 0, Phase.MIXED: 0, Phase.PREFILL: 0}
    tokens = {Phase.DECODE: 0, Phase.MIXED: 0, Phase.PREFILL: 0}
    flops = {Phase.DECODE: 0, Phase.MIXED: 0, Phase.PREFILL: 0}
    step_flops = getattr(getattr(getattr(engine, "runner", None), "model", None), "step_flops", None)  # what the parts say a step costs
    steps = 0
    t0 = time.perf_counter()
    while engine.has_unfinished and (max_steps is None or steps < max_steps):
        with mark("step"):
            t = time.perf_counter()
            batch = engine.step()
            t = time.perf_counter() - t
        steps += 1
        if batch is None:
            continue
        times[batch.phase].append(t)
        rows[batch.phase] += len(batch.rows)
        tokens[batch.phase] += batch.num_tokens
        if step_flops is not None:
            flops[batch.phase] += step_flops([(n, s) for _, s, n in batch.rows])
    span = time.perf_counter() - t0

    def kind(p):
        ts = times[p]
        if not ts:
            return {"steps": 0}
        return {"steps": len(ts), "median_ms": round(statistics.median(ts) * 1e3, 4), "mean_ms": round(sum(ts) / len(ts) * 1e3, 4),
                "mean_rows": round(rows[p] / len(ts), 2), "mean_tokens": round(tokens[p] / len(ts), 2),
                "mean_flops": flops[p] / len(ts)}

    return {"seconds": span, "steps": steps, "decode": kind(Phase.DECODE), "mixed": kind(Phase.MIXED), "prefill": kind(Phase.PREFILL)}
