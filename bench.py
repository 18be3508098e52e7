"""Decode throughput of the engine on one MI355X: Qwen3-0.6B-shaped model, random weights,
bfloat16, batch 8 at a context of 4,096 tokens per request, 16-token pages.

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the engine (schedule, one pass of the model over the batch's last
tokens, sampling on the device, one read-back of the tokens, which the engine waits for one step
after the launch). Requests are prefilled through the
same step function in portions of 2,048 tokens; the timed steps are the last K before every
request reaches the context length. One JSON line is printed, with ``value`` = decoded tokens per
second, plus the prefill rate of one 2,048-token prompt, the decode step's share of the HBM
roofline, and decode rates at batch 1 and 64.

Peaks: MI355X's published 8 TB/s HBM and 2.5 PFLOP/s dense bf16 (157.3 TFLOP/s float32). Beside them the
line carries ``measured_peaks``: what this box gives a streaming read of 1 GiB and the engine's bfloat16
product at n = 4096, and the decode step's bytes per second as a share of that read rate.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--preset", default="0.6B")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the preset has (reported in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill measurement")
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
    from miniserve_amd.loading import random_model

    cfg = preset(args.preset)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    model = random_model(cfg, seed=0, dtype=args.dtype, device="cuda:0")
    vocab = cfg["vocab_size"]
    gen = torch.Generator().manual_seed(0)

    def say(msg):
        print(f"[bench] {msg}", file=sys.stderr, flush=True)

    def prompts(n, length):
        return [torch.randint(0, min(vocab, 150000), (length,), generator=gen).tolist() for _ in range(n)]

    def decode_run(batch: int, steps: int, warmup: int):
        """Decode ``warmup + steps`` tokens for ``batch`` requests ending at the context length;
        returns (seconds for the timed steps, mean context over them, engine)."""
        total = warmup + steps
        # Decoding requests keep decoding while later ones are still prefilled (about two steps per
        # request at a step budget of 2,048 tokens): prompts are shortened by that much, so that the
        # longest sequence ends at the context length.
        lead = 2 * batch
        plen = args.context - total - lead
        eng = Engine(model, max_running=batch, kv_pool_tokens=batch * (args.context + 32), chunked_prefill_size=2048,
                     decode_graph=not args.no_graph)
        reqs = [eng.add_request(p, SamplingParams(max_new_tokens=total + lead + 8)) for p in prompts(batch, plen)]
        say(f"batch {batch}: prefilling {batch} x {plen} tokens")
        last = time.time()
        while not all(r.state is RequestState.DECODE for r in reqs):
            eng.step()
            if time.time() - last > 20:
                last = time.time()
                say(f"  prefill: {sum(r.cache.num_tokens for r in reqs if r.cache)} tokens in the cache")
        say(f"batch {batch}: decoding {warmup} + {steps} steps at contexts {min(r.seq_len for r in reqs)}..{max(r.seq_len for r in reqs)}")
        for _ in range(warmup):
            eng.step()
        torch.cuda.synchronize()
        ctx0 = sum(r.seq_len for r in reqs) / batch
        t0 = time.perf_counter()
        for _ in range(steps):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert all(r.state is RequestState.DECODE for r in reqs), "a request ended inside the timed steps"
        mean_ctx = ctx0 + (steps - 1) / 2
        for r in reqs:
            eng.abort(r.rid)
        return dt, mean_ctx, eng

    if args.prefill_only:
        dt, mean_ctx, eng = 1.0, 0.0, None
    else:
        dt, mean_ctx, eng = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    weight_bytes = model.decode_read_bytes()
    kv_bytes = args.batch * mean_ctx * (eng.runner.pool.bytes_per_token() if eng else 0)
    achieved = (weight_bytes + kv_bytes) / (dt / args.steps) / 1e9
    del eng

    out = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen3-{args.preset} shape, context {args.context})",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights, random token ids)",
        "config": {
            "model": f"Qwen3-{args.preset}-shaped", "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "single GPU", "layers": cfg["num_hidden_layers"], "layers_full": full_layers,
            "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": vocab,
            "page_size": 16, "decode_graph": not args.no_graph, "overlap": True,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }

    if not args.no_points:
        # Prefill of one 2,048-token prompt in one step (logits at the last position).
        from miniserve_amd.engine.runner import ModelRunner

        T, C = args.prefill_tokens, args.prefill_cached
        runner = ModelRunner(model, kv_pool_tokens=4 * T + C + 64, max_running=4)
        times = []
        for i in range(4):
            rc = runner.acquire()
            ids = prompts(1, T)[0]
            for at in range(0, C, 2048):
                runner.step([StepRow(rc, prompts(1, min(2048, C - at))[0], [])])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            runner.step([StepRow(rc, ids, [T - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            runner.release(rc)
        pre = min(times[1:])
        L, H, I = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"]
        Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
        linear = 2 * T * L * (H * (Hq + 2 * Hkv) * D + Hq * D * H + 3 * H * I) + 2 * H * vocab
        attn = 2 * T * (T + 2 * C) * D * Hq * L  # causal: QK^T and PV over half the square each, and over the cached keys
        flops = linear + attn
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        out["prefill"] = {"value": round(T / pre, 1), "tokens": T, "ms": round(pre * 1e3, 3),
                          "frac": round(flops / pre / peak, 4)}
        if C:
            out["prefill"]["cached"] = C
        del runner
        points = {}
        for b, steps in ((1, 64), (64, 24)) if not args.prefill_only else ():
            d, _, e = decode_run(b, steps, 8)
            points[f"decode_b{b}"] = round(b * steps / d, 1)
            del e
        out["points"] = points

    if not args.no_points or args.prefill_only:
        # What this box gives beside the published peaks (the same kernels as `python -m miniserve_amd roofline`).
        from miniserve_amd.kernels import ops

        def median_ms(fn, repeats=5):
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
        del buf
        x = torch.randn((4096, 4096), device="cuda:0").to(torch.bfloat16)
        w = torch.randn((4096, 4096), device="cuda:0").to(torch.bfloat16)
        rate = 2 * 4096**3 / median_ms(lambda: ops.linear(x, w, out_dtype=torch.bfloat16)) / 1e9
        out["measured_peaks"] = {"read_GBps": round(read, 1), "gemm_bf16_4096_TFLOPs": round(rate, 1),
                                 "decode_frac_of_read": round(achieved / read, 4)}

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
