"""``python -m miniserve_amd <command>``: generate, stress, random-weights.

* ``generate``: token ids in, token ids out, through ``Engine.generate``.
* ``stress``: the reference's offline stress run (miniserve/tools/stress.py:28-84): random-length
  requests of random ids, a JSON report (decode-only and mixed step times apart, the engine's effective
  configuration read back from it, the runtime), exit 1 unless every request finished and every page is back.
* ``random-weights``: write a model folder with random weights.
"""

from __future__ import annotations

import argparse
import json
import random
import sys
import time


def _add_model_args(ap: argparse.ArgumentParser) -> None:
    from .config.presets import PRESETS

    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", "--model-dir", dest="model", help="folder with config.json and *.safetensors")
    src.add_argument("--preset", choices=sorted(PRESETS), help="a named shape with random weights")
    ap.add_argument("--weights-seed", type=int, default=0, help="seed of the random weights of --preset")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--device", default="cuda:0")


def _build_engine(args):
    from .config.presets import preset
    from .engine.cli import engine_kwargs
    from .engine.engine import Engine
    from .loading import load_model, random_model

    if args.model:
        model = load_model(args.model, args.dtype, args.device)
    else:
        model = random_model(preset(args.preset), args.weights_seed, args.dtype, args.device)
    return Engine(model, **engine_kwargs(args))


def cmd_generate(args) -> int:
    from .engine.request import SamplingParams

    eng = _build_engine(args)
    vocab = eng.runner.model.vocab_size
    if args.prompt_ids:
        prompts = [[int(t) for t in p.split(",")] for p in args.prompt_ids]
    else:
        rng = random.Random(args.workload_seed)
        prompts = [[rng.randrange(min(vocab, 150000)) for _ in range(args.prompt_len)] for _ in range(args.num_prompts)]
    params = SamplingParams(args.max_new_tokens, frozenset(args.stop_token_ids), args.temperature, args.top_p, args.sample_seed)
    t0 = time.time()
    outs = eng.generate(prompts, params)
    dt = time.time() - t0
    print(json.dumps({"outputs": outs, "seconds": round(dt, 4), "steps": eng.num_steps,
                      "preemptions": eng.scheduler.num_preemptions}))
    return 0


def cmd_stress(args) -> int:
    from .engine.request import SamplingParams

    eng = _build_engine(args)
    vocab = eng.runner.model.vocab_size
    rng = random.Random(args.workload_seed)
    reqs = []
    for _ in range(args.num_requests):
        n = rng.randint(*args.prompt_len)
        new = rng.randint(*args.max_new_tokens)
        ids = [rng.randrange(min(vocab, 150000)) for _ in range(n)]
        reqs.append(eng.add_request(ids, SamplingParams(new, temperature=args.temperature, top_p=args.top_p)))
    from .measurement.offline import run_to_completion
    from .measurement.sidecar import sidecar

    ran = run_to_completion(eng, args.max_steps)
    dt = ran["seconds"]
    finished = sum(r.state.value == "finished" for r in reqs)
    tokens = sum(len(r.output_ids) for r in reqs)
    report = {
        "requests": len(reqs), "finished": finished, "steps": ran["steps"], "output_tokens": tokens,
        "seconds": round(dt, 3), "tokens_per_second": round(tokens / dt, 1) if dt > 0 else None,
        "preemptions": eng.scheduler.num_preemptions, "dropped_tokens": eng.dropped_tokens, "idle": eng.runner.cache.idle,
        # decode-only steps apart from steps that carry portions of prompts
        "decode_steps": ran["decode"], "mixed_steps": ran["mixed"], "prefill_steps": ran["prefill"],
        "stats": dict(eng.scheduler.stats),
    }
    report.update(sidecar(eng))
    print(json.dumps(report))
    return 0 if finished == len(reqs) and eng.runner.cache.idle else 1


def cmd_roofline(args) -> int:
    """What this GPU gives beside its published peaks, measured with the engine's own kernels: the rate
    of a streaming read and of a streaming copy over ``--mib`` MiB (the reference measures both at
    1 GiB, bench/roofline.py:85-121), and the bfloat16 matrix product's rate at n = 4096 and 8192
    (bench/roofline.py:184-198). Times are medians of ``--repeats`` runs by device events."""
    import torch

    from .kernels import ops

    dev = torch.device(args.device)
    torch.cuda.set_device(dev)

    def median_ms(fn):
        fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(args.repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1))
        return sorted(times)[len(times) // 2]

    n = args.mib << 20
    src = torch.empty((n,), dtype=torch.uint8, device=dev)
    dst = torch.empty((n,), dtype=torch.uint8, device=dev)
    src.random_(0, 256)
    report = {"device": torch.cuda.get_device_name(dev), "mib": args.mib, "repeats": args.repeats}
    with ops.stream_scope():
        report["read_GBps"] = round(n / median_ms(lambda: ops.measure_read(src, args.blocks)) / 1e6, 1)
        report["copy_GBps"] = round(2 * n / median_ms(lambda: ops.measure_copy(src, dst, args.blocks)) / 1e6, 1)
        assert torch.equal(src[: 1 << 20], dst[: 1 << 20]) and torch.equal(src[-(1 << 20) :], dst[-(1 << 20) :])
        del src, dst
        gemm = {}
        for size in (4096, 8192):
            x = torch.randn((size, size), device=dev).to(torch.bfloat16)
            w = torch.randn((size, size), device=dev).to(torch.bfloat16)
            ms = median_ms(lambda: ops.linear(x, w, out_dtype=torch.bfloat16))
            gemm[str(size)] = round(2 * size**3 / ms / 1e9, 1)
        report["gemm_bf16_TFLOPs"] = gemm
    report["published"] = {"hbm_GBps": 8000.0, "bf16_TFLOPs": 2500.0}
    print(json.dumps(report))
    return 0


def main(argv=None) -> int:
    from .engine.cli import add_engine_args

    ap = argparse.ArgumentParser(prog="python -m miniserve_amd")
    sub = ap.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate token ids for prompts of token ids")
    _add_model_args(g)
    add_engine_args(g)
    g.add_argument("--prompt-ids", action="append", help="comma-separated token ids; repeat for several prompts")
    g.add_argument("--prompt-len", type=int, default=16, help="length of the random prompts used without --prompt-ids")
    g.add_argument("--num-prompts", type=int, default=1)
    g.add_argument("--workload-seed", type=int, default=0)
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--stop-token-ids", type=int, nargs="*", default=[])
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--sample-seed", type=int, default=None, help="sampling seed of every request (default: from --seed)")
    g.set_defaults(fn=cmd_generate)

    s = sub.add_parser("stress", help="random-length offline run with a JSON report")
    _add_model_args(s)
    add_engine_args(s)
    s.add_argument("--num-requests", type=int, default=64)
    s.add_argument("--prompt-len", type=int, nargs=2, default=[16, 512], metavar=("MIN", "MAX"))
    s.add_argument("--max-new-tokens", type=int, nargs=2, default=[1, 128], metavar=("MIN", "MAX"))
    s.add_argument("--workload-seed", type=int, default=0)
    s.add_argument("--temperature", type=float, default=0.0)
    s.add_argument("--top-p", type=float, default=1.0)
    s.add_argument("--max-steps", type=int, default=100000)
    s.set_defaults(fn=cmd_stress)

    r = sub.add_parser("roofline", help="measured read / copy bandwidth and bfloat16 matrix-product rate of this GPU")
    r.add_argument("--device", default="cuda:0")
    r.add_argument("--mib", type=int, default=1024, help="size of the buffers that are read and copied")
    r.add_argument("--blocks", type=int, default=4096, help="blocks of the streaming kernels")
    r.add_argument("--repeats", type=int, default=9)
    r.set_defaults(fn=cmd_roofline)

    w = sub.add_parser("random-weights", help="write a model folder with random weights")
    w.add_argument("rest", nargs=argparse.REMAINDER)
    w.set_defaults(fn=None)

    args = ap.parse_args(argv)
    if args.command == "random-weights":
        from .weights.random_init import main as rw_main

        return rw_main(args.rest)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
