"""What an engine is actually running, read back from the live objects: several settings that matter
most for a measurement are decided inside the engine (the pool's size, the step budget's default,
which graphs exist), not on the command line. Same idea and keys as the reference where it has them
(miniserve/engine/describe.py:22-67)."""

from __future__ import annotations

import subprocess
from pathlib import Path


def engine_description(engine) -> dict:
    """The engine's effective configuration as it ended up."""
    runner, sched = engine.runner, engine.scheduler
    graphs = getattr(runner, "graphs", None)
    cache = runner.cache
    model = getattr(runner, "model", None)
    spec = getattr(model, "spec", None)
    out = dict(
        architecture=getattr(spec, "architecture", None),
        dtype=str(getattr(model, "dtype", "")).removeprefix("torch.") or None,
        max_running=sched.max_running,
        max_prefill_tokens=sched.max_prefill_tokens,
        chunked_prefill_size=sched.chunked_prefill_size,
        schedule_policy=sched.policy.name,
        overlap=engine.overlap,
        page_size=cache.page_size,
        kv_pool_pages=cache.total_pages(),  # per layer group
        kv_pool_tokens=[n * cache.page_size for n in cache.total_pages()],
        cache_groups=[dict(slots=len(g.slots), window=g.window, planes=[(p.name, p.heads, p.width) for p in g.planes])
                      for g in cache.layout.groups],
        state_slots=cache.state_slots.num_slots,
        block_backend=cache.allocators[0].backend if cache.allocators else None,
        decode_graph=graphs is not None,
        decode_graph_buckets=None if graphs is None else list(graphs.buckets),
        decode_graphs_captured=None if graphs is None else sorted(graphs.captured),
        max_position=getattr(spec, "max_position", None),
    )
    profile = getattr(runner, "kv_profile", None)
    if profile:
        out["kv_profile"] = dict(profile)
    return out


def runtime_description() -> dict:
    """The software and the device underneath, for the same record."""
    import torch

    def git(*args: str):
        try:
            root = Path(__file__).resolve().parents[2]
            return subprocess.run(["git", "-C", str(root), *args], capture_output=True, text=True, check=True, timeout=10).stdout.strip()
        except Exception:  # noqa: BLE001  (a checkout is not always there)
            return None

    props = torch.cuda.get_device_properties(0) if torch.cuda.is_available() else None
    from ..kernels import build

    return dict(
        torch=torch.__version__,
        hip=getattr(torch.version, "hip", None),
        gpu=None if props is None else props.name,
        gpu_arch=None if props is None else getattr(props, "gcnArchName", None),
        gpu_memory_bytes=None if props is None else props.total_memory,
        compute_units=None if props is None else props.multi_processor_count,
        kernel_library=build.kernel_library_name(),
        git_commit=git("rev-parse", "HEAD"),
        git_dirty=bool(git("status", "--porcelain", "--untracked-files=no")),
    )
