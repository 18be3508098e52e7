"""What the command-line entry points promise without a GPU: ``bench.py`` refuses more than one GPU
with one line and exit code 2, ``bin/trace_run`` documents its options, and the kernel library's
sources are all found by the build."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def run(*args):
    return subprocess.run([sys.executable, *map(str, args)], capture_output=True, text=True, timeout=120, cwd=ROOT)


def test_bench_refuses_more_than_one_gpu():
    p = run(ROOT / "bench.py", "--gpus", "2", "--steps", "1", "--warmup", "0")
    assert p.returncode == 2
    lines = [line for line in p.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_trace_run_names_its_options():
    p = run(ROOT / "bin" / "trace_run", "--help")
    assert p.returncode == 0
    for opt in ("--model", "--dtype", "--out", "--max-tokens"):
        assert opt in p.stdout
    assert "bfloat16" in p.stdout and "float32" in p.stdout


def test_build_finds_every_source():
    from miniserve_amd.kernels import build

    names = {s.name for s in build.hip_sources()}
    assert {"attention.hip", "attention_decode.hip", "attention_prefill.hip", "elementwise.hip", "gemm_bf16.hip", "measure.hip",
            "gemm_f32.hip", "sampling.hip"} <= names
    assert [s.name for s in build.cpp_sources()] == ["block_core.cpp"]
    assert "-packed-fp32-ops" in build.HIP_FLAGS, "packed float32 instructions stay off"


@pytest.mark.gpu
def test_bench_line_on_a_tiny_shape():
    """The benchmark's one JSON line with a tiny preset: every key of the contract, the flat config of
    at most 20 keys, the prefill and roofline records, the batch 1 and 64 points, the sidecar."""
    p = run(ROOT / "bench.py", "--preset", "tinyE", "--batch", "2", "--context", "512", "--steps", "4", "--warmup", "2",
            "--prefill-tokens", "128", "--warmup-seconds", "0.02", "--warmup-most-seconds", "0.05")
    assert p.returncode == 0, p.stderr[-2000:]
    line = json.loads(p.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "prefill", "points"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 4 and line["warmup"] == 2 and line["value"] > 0
    assert len(line["config"]) <= 20 and all(not isinstance(v, (dict, list)) for v in line["config"].values())
    assert line["config"]["layers"] == line["config"]["layers_full"] == 3
    assert set(line["roofline"]) == {"bound", "achieved", "peak", "unit", "frac"} and line["roofline"]["peak"] == 8000.0
    assert line["prefill"]["tokens"] == 128 and line["prefill"]["value"] > 0
    assert set(line["points"]) == {"decode_b1", "decode_b1_frac", "decode_b64", "decode_b64_frac"}
    assert line["config"]["warmup_steps_run"] == 2
    side = line["sidecar"]
    assert side["runtime"]["torch"] and side["runtime"]["kernel_library"].startswith("libmsamd_kernels_")
    assert side["engine"]["kv_pool_tokens"] == [2 * (512 + 32)] * 2 and side["engine"]["decode_graph"] is True
    assert side["engine"]["chunked_prefill_size"] == 2048 and side["warmup"]["steps"] == 2
    # after the warm-up steps the last one is repeated, at least for the time asked for and until the clock is steady
    assert side["warmup"]["repeats_of_the_last_step"] >= 8 and side["warmup"]["held_seconds"] >= 0.02
    assert side["warmup"]["clock_steady"] in (True, False, None)
    assert "copy_GBps" in line["measured_peaks"] and line["measured_peaks"]["copy_GBps"] > 100
    assert side["conditions"]["power_limit_w"] is None or 100 < side["conditions"]["power_limit_w"] < 5000


@pytest.mark.gpu
def test_the_monitor_reads_a_loaded_gpu():
    """The readings themselves, not their arithmetic: under a sustained matrix product the shader clock is
    far above its idle value, the socket draws a plausible power (a scale wrong by a thousand shows), the
    memory clock and the temperatures are there, and the limits name a power limit above what is drawn."""
    import time

    import torch

    from miniserve_amd.kernels import ops
    from miniserve_amd.measurement import GpuMonitor

    x = torch.randn((8192, 8192), device="cuda:0").to(torch.bfloat16)
    w = torch.randn((8192, 8192), device="cuda:0").to(torch.bfloat16)

    def work():
        for _ in range(10):
            ops.linear(x, w, out_dtype=torch.bfloat16)
        torch.cuda.synchronize()

    with GpuMonitor(interval_s=0.02) as g:
        t0 = time.monotonic()
        out = g.warm_until_steady(work, least_s=1.0, most_s=5.0)
        busy = g.window(since=t0 + 1.2)  # the first refresh after the load began may still mix idle and load
        limits = g.conditions()
    assert out["steady"] is not None, "the clock could be read often enough to decide"
    assert busy["samples"] >= 2, "the firmware refreshes its figures about once a second"
    assert busy["sclk_mhz"]["mean"] > 1000, busy
    assert 50 < busy["power_w"]["mean"] < 2000 and busy["power_w"]["max"] < 2000, busy
    assert busy["mclk_mhz"]["mean"] > 500 and 10 < busy["temp_c"]["mean"] < 120, busy
    assert busy["busy_pct"]["max"] > 50, busy
    assert limits["power_limit_w"] is not None and limits["power_limit_w"] >= busy["power_w"]["mean"] * 0.9, limits
    assert limits["sclk_range_mhz"] is not None and limits["sclk_range_mhz"][1] >= busy["sclk_mhz"]["max"] * 0.95


@pytest.mark.gpu
def test_roofline_reports_measured_rates():
    p = run("-m", "miniserve_amd", "roofline", "--mib", "64", "--repeats", "3")
    assert p.returncode == 0, p.stderr[-2000:]
    report = json.loads(p.stdout.strip().splitlines()[-1])
    assert report["read_GBps"] > 100 and report["copy_GBps"] > 100
    assert set(report["gemm_bf16_TFLOPs"]) == {"4096", "8192"} and all(v > 10 for v in report["gemm_bf16_TFLOPs"].values())
    assert report["published"] == {"hbm_GBps": 8000.0, "bf16_TFLOPs": 2500.0}
