"""Decode throughput of the engine on one MI355X: Qwen3-0.6B-shaped model, random weights,
bfloat16, batch 8 at a context of 4,096 tokens per request, 16-token pages.

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the engine (schedule, one pass of the model over the batch's last
tokens, sampling on the device, one read-back of the tokens, which the engine waits for one step
after the launch). Requests are prefilled through the same step function in portions of 2,048 tokens;
the timed steps are the last K before every request reaches the context length. Before them run W
untimed decode steps, and then the last of them is run again and again on the same inputs (the same
kernels at the same context; nothing advances, so the timed steps still end at the context length)
for at least ``--warmup-seconds`` and until the GPU's shader clock has stopped moving, at most
``--warmup-most-seconds``; what the clock, the power and the temperatures did meanwhile is in ``sidecar``.

One JSON line is printed. ``value`` = decoded tokens per second of the headline point. Beside it:
``prefill`` (one 2,048-token prompt in one step; median of five; its flops are what the model's parts say
of themselves), ``roofline`` (the decode step's bytes,
every weight once plus the live requests' cache, over its time, against the published 8 TB/s),
``points`` (decode at batch 1 and 64 of the same shape; unless ``--no-extra``, decode at batch 8 behind
32,768 tokens and a prompt of 8,192 tokens in one step, the Qwen3-8B shape's decode at batch 1 / 8 / 64 / 128 /
256 and at batch 32 behind 16,384 tokens, its prefill and the same two further lengths, and the Qwen3-32B
shape's continuous batching of 64 requests with 2,048-token prompts under a 512-token step budget,
decode-only and mixed steps timed apart, its decode at batch 1 / 8 / 64 and its 2,048-token prefill, each
with its share of the roofline), ``measured_peaks`` (what this box gives a streaming read
and the engine's bfloat16 product) and ``sidecar`` (device, clocks and power while the headline point
ran, versions, commit, the engine's effective configuration).

Peaks: MI355X's published 8 TB/s HBM and 2.5 PFLOP/s dense bf16 (157.3 TFLOP/s float32).
"""

from __future__ import annotations

import argparse
import gc
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def say(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--warmup-seconds", type=float, default=0.3,
                    help="after the warm-up steps, repeat the last of them for at least this long and until the clock is steady")
    ap.add_argument("--warmup-most-seconds", type=float, default=4.5,
                    help="give up waiting for a steady clock after this long (the firmware reports about once a second)")
    ap.add_argument("--preset", default="0.6B")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the preset has (reported in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points, the prefill and the extra shapes")
    ap.add_argument("--no-extra", action="store_true", help="skip the 8B and 32B shapes")
    ap.add_argument("--no-graph", action="store_true", help="run decode steps eagerly")
    ap.add_argument("--prefill-only", action="store_true", help="measure only the prefill (for profiling)")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="tokens of the timed prefill step")
    ap.add_argument("--prefill-cached", type=int, default=0,
                    help="tokens of the same sequence already in the cache when the timed step runs (fed untimed, 2,048 a step)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    from miniserve_amd.config.presets import preset
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.engine import Engine
    from miniserve_amd.engine.request import RequestState, SamplingParams
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import random_model
    from miniserve_amd.measurement import GpuMonitor, measured_region, sidecar
    from miniserve_amd.measurement.offline import run_to_completion

    dt_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    gen = torch.Generator().manual_seed(0)

    def prompts(vocab, n, length):
        return [torch.randint(0, min(vocab, 150000), (length,), generator=gen).tolist() for _ in range(n)]

    def make(name, layers=None):
        cfg = preset(name)
        full = cfg["num_hidden_layers"]
        if layers:
            cfg["num_hidden_layers"] = layers
        say(f"building the {name} shape ({cfg['num_hidden_layers']} of {full} layers, {args.dtype})")
        return cfg, full, random_model(cfg, seed=0, dtype=args.dtype, device="cuda:0")

    def decode_run(model, cfg, batch, steps, warmup, describe=False, context=None):
        """Decode ``steps`` timed tokens for ``batch`` requests ending at the context length, after the
        warm-up; returns a dict with the rate, the step time and the step's share of the roofline. With
        ``describe`` (the headline point) the warm-up waits for a steady clock, and the last step is kept
        running after the timed ones until the firmware has reported on the device once more."""
        context = context or args.context
        warm_steps = max(warmup, 1)
        total = warm_steps + steps
        # Decoding requests keep decoding while later ones are still prefilled (a step per 2,048 prompt
        # tokens of each): prompts are shortened by that much, so that the longest sequence ends at the
        # context length.
        lead = batch * max(2, math.ceil((context - total) / 2048))
        plen = context - total - lead
        if plen < 1:
            raise SystemExit(f"context {context} is too short for {total} decode steps")
        eng = Engine(model, max_running=batch, kv_pool_tokens=batch * (context + 32), chunked_prefill_size=2048,
                     decode_graph=not args.no_graph)
        reqs = [eng.add_request(p, SamplingParams(max_new_tokens=total + lead + 8)) for p in prompts(cfg["vocab_size"], batch, plen)]
        say(f"batch {batch}: prefilling {batch} x {plen} tokens")
        last = time.time()
        while not all(r.state is RequestState.DECODE for r in reqs):
            eng.step()
            if time.time() - last > 20:
                last = time.time()
                say(f"  prefill: {sum(r.cache.num_tokens for r in reqs if r.cache)} tokens in the cache")
        say(f"batch {batch}: decoding {warm_steps} + {steps} steps at contexts {min(r.seq_len for r in reqs)}..{max(r.seq_len for r in reqs)}")
        torch.cuda.synchronize()
        w0 = time.perf_counter()
        for _ in range(warm_steps):
            eng.step()
        torch.cuda.synchronize()

        def hold():  # the latest step again, a few times: the device stays at the step's load, the context stays put
            for _ in range(8):
                eng.runner.repeat_last_step()
            torch.cuda.synchronize()

        most = max(args.warmup_seconds, args.warmup_most_seconds) if describe else args.warmup_seconds
        held = monitor.warm_until_steady(hold, args.warmup_seconds, most)
        warm_s = time.perf_counter() - w0
        monitor.interval_s = 0.25  # fewer readings while the host is being timed
        ctx0 = sum(r.seq_len for r in reqs) / batch
        t_mark = monitor.read_now()
        with measured_region(f"decode b{batch}"):
            t0 = time.perf_counter()
            for _ in range(steps):
                eng.step()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        assert all(r.state is RequestState.DECODE for r in reqs), "a request ended inside the timed steps"
        mean_ctx = ctx0 + (steps - 1) / 2
        step_bytes = model.decode_read_bytes() + batch * mean_ctx * eng.runner.pool.bytes_per_token()
        out = {"tok_s": batch * steps / dt, "ms_per_step": dt / steps * 1e3, "mean_ctx": mean_ctx,
               "achieved_gbs": step_bytes / (dt / steps) / 1e9, "warmup_steps": warm_steps, "warmup_s": round(warm_s, 3),
               "held": held, "since": t_mark}
        monitor.interval_s = 0.05
        if describe:  # the timed steps are over in a few hundredths of a second: no refresh falls inside them
            monitor.hold_until_refresh(hold)
        out["until"] = monitor.read_now()
        if describe:
            out["sidecar"] = sidecar(eng)
        for r in reqs:
            eng.abort(r.rid)
        del eng
        return out

    def prefill_run(model, cfg, T, C, repeats=5):
        """One prompt of ``T`` tokens in one step (logits at the last position), ``C`` tokens of the same
        sequence already cached; the median of ``repeats`` timed runs after one untimed."""
        runner = ModelRunner(model, kv_pool_tokens=4 * T + C + 64, max_running=4)
        vocab = cfg["vocab_size"]
        times = []
        for i in range(repeats + 1):
            rc = runner.acquire()
            ids = prompts(vocab, 1, T)[0]
            for at in range(0, C, 2048):
                runner.step([StepRow(rc, prompts(vocab, 1, min(2048, C - at))[0], [])])
            torch.cuda.synchronize()
            with measured_region("prefill") if i else measured_region("prefill (untimed)"):
                t0 = time.perf_counter()
                runner.step([StepRow(rc, ids, [T - 1])])
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
            runner.release(rc)
        pre = statistics.median(times[1:])
        # every matrix product of the T tokens, both attention products over each (query, visible key) pair, the head once
        out = {"value": round(T / pre, 1), "tokens": T, "ms": round(pre * 1e3, 3),
               "frac": round(model.step_flops([(T, C)]) / pre / PEAK_FLOPS[dt_name], 4)}
        if C:
            out["cached"] = C
        del runner
        return out

    def continuous_run(model, cfg, requests=64, prompt_len=2048, new_tokens=512, budget=512):
        """The reference's offline workload for its largest model: all requests at once, prompts cut into
        portions under a step budget and mixed with decoding requests. Decode-only and mixed steps are
        timed apart; a mixed step's flops are what the model's parts say of its rows (attention included)."""
        eng = Engine(model, max_running=requests, kv_pool_tokens=requests * (prompt_len + new_tokens + 32),
                     chunked_prefill_size=budget, decode_graph=not args.no_graph)
        for p in prompts(cfg["vocab_size"], requests, prompt_len):
            eng.add_request(p, SamplingParams(max_new_tokens=new_tokens))
        with measured_region("continuous batching"):
            ran = run_to_completion(eng)
        torch.cuda.synchronize()
        assert eng.runner.cache.idle
        weights = model.decode_read_bytes()
        per_tok = eng.runner.pool.bytes_per_token()
        out = {"tok_s": requests * new_tokens / ran["seconds"], "seconds": ran["seconds"], "preemptions": eng.scheduler.num_preemptions}
        d, m = ran["decode"], ran["mixed"]
        if d["steps"]:
            ctx = prompt_len + new_tokens / 2
            out["decode_step_ms"] = d["median_ms"]
            out["decode_rows"] = d["mean_rows"]
            out["decode_frac"] = (weights + d["mean_rows"] * ctx * per_tok) / (d["median_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS
        if m["steps"]:
            out["mixed_step_ms"] = m["median_ms"]
            out["mixed_tokens"] = m["mean_tokens"]
            out["mixed_frac_flops"] = m["mean_flops"] / (m["median_ms"] * 1e-3) / PEAK_FLOPS[dt_name]
            out["mixed_frac_hbm"] = weights / (m["median_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS
        del eng
        return out

    cfg, full_layers, model = make(args.preset, args.layers)
    vocab = cfg["vocab_size"]
    side = {}
    monitor = GpuMonitor().start()  # polls from here to the end of the run
    if args.prefill_only:
        head = {"tok_s": 0.0, "ms_per_step": 0.0, "achieved_gbs": 0.0, "mean_ctx": 0.0, "warmup_steps": 0}
    else:
        head = decode_run(model, cfg, args.batch, args.steps, args.warmup, describe=True)
        side = head.pop("sidecar")
        side["warmup"] = {"steps": head["warmup_steps"], "seconds": head["warmup_s"], "repeats_of_the_last_step": 8 * head["held"]["calls"],
                          "held_seconds": head["held"]["seconds"], "refreshes_seen": head["held"]["refreshes"],
                          "clock_steady": head["held"]["steady"]}
        # the firmware's first report after the timed steps, taken while their last step was kept running
        side["gpu_at_timed_steps"] = monitor.window(head["since"], head["until"])
    achieved = head["achieved_gbs"]

    out = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen3-{args.preset} shape, context {args.context})",
        "value": round(head["tok_s"], 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt_name, "data": "synthetic (random weights, random token ids)",
        "config": {
            "model": f"Qwen3-{args.preset}-shaped", "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "single GPU", "layers": cfg["num_hidden_layers"], "layers_full": full_layers,
            "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": vocab,
            "page_size": 16, "decode_graph": not args.no_graph, "overlap": True, "warmup_steps_run": head["warmup_steps"],
            "mean_context_timed": round(head["mean_ctx"], 1),
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }

    if not args.no_points:
        out["prefill"] = prefill_run(model, cfg, args.prefill_tokens, args.prefill_cached)
        points = {}
        for b, steps in ((1, 64), (64, 24)) if not args.prefill_only else ():
            r = decode_run(model, cfg, b, steps, 8)
            points[f"decode_b{b}"] = round(r["tok_s"], 1)
            points[f"decode_b{b}_frac"] = round(r["achieved_gbs"] / HBM_PEAK_GBS, 4)
        out["points"] = points

    if not args.no_points or args.prefill_only:
        # What this box gives beside the published peaks (the same kernels as `python -m miniserve_amd roofline`).
        from miniserve_amd.kernels import ops

        def median_ms(fn, repeats=9, warm=3):
            for _ in range(warm):
                fn()
            torch.cuda.synchronize()
            times = []
            for _ in range(repeats):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                e1.synchronize()
                times.append(e0.elapsed_time(e1))
            return sorted(times)[len(times) // 2]

        n = 1 << 30
        buf = torch.empty((n,), dtype=torch.uint8, device="cuda:0").random_(0, 256)
        read = n / median_ms(lambda: ops.measure_read(buf)) / 1e6
        dst = torch.empty_like(buf)
        copy = 2 * n / median_ms(lambda: ops.measure_copy(buf, dst)) / 1e6  # bytes read plus bytes written
        del buf, dst
        rates = {}
        for n in (4096, 8192):
            x = torch.randn((n, n), device="cuda:0").to(torch.bfloat16)
            w = torch.randn((n, n), device="cuda:0").to(torch.bfloat16)
            rates[n] = 2 * n**3 / median_ms(lambda: ops.linear(x, w, out_dtype=torch.bfloat16)) / 1e9
            del x, w
        out["measured_peaks"] = {"read_GBps": round(read, 1), "copy_GBps": round(copy, 1), "gemm_bf16_4096_TFLOPs": round(rates[4096], 1),
                                 "gemm_bf16_8192_TFLOPs": round(rates[8192], 1),
                                 "decode_frac_of_read": round(achieved / read, 4)}

    if not (args.no_points or args.no_extra or args.prefill_only) and args.preset == "0.6B" and not args.layers:
        points = out["points"]
        # further context lengths: decode behind 32,768 tokens, a prompt of 8,192 in one step
        r = decode_run(model, cfg, 8, 24, 8, context=32768)
        points["decode_b8_ctx32768"] = round(r["tok_s"], 1)
        points["decode_b8_ctx32768_frac"] = round(r["achieved_gbs"] / HBM_PEAK_GBS, 4)
        p = prefill_run(model, cfg, 8192, 0, repeats=3)
        points["prefill_8192"] = p["value"]
        points["prefill_8192_frac"] = p["frac"]
        del model
        gc.collect()
        torch.cuda.empty_cache()
        cfg8, _, m8 = make("8B")
        for b, steps in ((1, 32), (8, 32), (64, 16)):
            r = decode_run(m8, cfg8, b, steps, 8)
            points[f"8B_decode_b{b}"] = round(r["tok_s"], 1)
            points[f"8B_decode_b{b}_frac"] = round(r["achieved_gbs"] / HBM_PEAK_GBS, 4)
        p8 = prefill_run(m8, cfg8, 2048, 0)
        points["8B_prefill_2048"] = p8["value"]
        points["8B_prefill_2048_frac"] = p8["frac"]
        r = decode_run(m8, cfg8, 8, 16, 8, context=32768)
        points["8B_decode_b8_ctx32768"] = round(r["tok_s"], 1)
        points["8B_decode_b8_ctx32768_frac"] = round(r["achieved_gbs"] / HBM_PEAK_GBS, 4)
        p8 = prefill_run(m8, cfg8, 8192, 0, repeats=3)
        points["8B_prefill_8192"] = p8["value"]
        points["8B_prefill_8192_frac"] = p8["frac"]
        # larger batches, and a batch behind 16,384 tokens
        for b, steps, ctx in ((128, 12, 4096), (256, 8, 4096), (32, 12, 16384)):
            r = decode_run(m8, cfg8, b, steps, 4, context=ctx)
            name = f"8B_decode_b{b}" + ("" if ctx == 4096 else f"_ctx{ctx}")
            points[name] = round(r["tok_s"], 1)
            points[name + "_frac"] = round(r["achieved_gbs"] / HBM_PEAK_GBS, 4)
        del m8
        gc.collect()
        torch.cuda.empty_cache()
        cfg32, _, m32 = make("32B")
        c = continuous_run(m32, cfg32)
        for k, v in c.items():
            points[f"32B_cont64_{k}"] = round(v, 4 if "frac" in k else 2)
        for b, steps in ((1, 12), (8, 12), (64, 8)):
            r = decode_run(m32, cfg32, b, steps, 4)
            points[f"32B_decode_b{b}"] = round(r["tok_s"], 1)
            points[f"32B_decode_b{b}_frac"] = round(r["achieved_gbs"] / HBM_PEAK_GBS, 4)
        p32 = prefill_run(m32, cfg32, 2048, 0, repeats=3)
        points["32B_prefill_2048"] = p32["value"]
        points["32B_prefill_2048_frac"] = p32["frac"]
        del m32
        gc.collect()
        torch.cuda.empty_cache()

    monitor.stop()
    if side:
        side["gpu_during_run"] = monitor.window()
        side["conditions"] = monitor.conditions()
        out["sidecar"] = side
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
