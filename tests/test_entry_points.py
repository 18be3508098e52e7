"""What the command-line entry points promise without a GPU: ``bench.py`` refuses more than one GPU
with one line and exit code 2, ``bin/trace_run`` documents its options, and the kernel library's
sources are all found by the build."""

from __future__ import annotations

import subprocess
import sys
from pathlib import Path

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
