"""What an engine is actually running, read back from the live objects: several settings that matter
most for a measurement are decided inside the engine (the pool's size, the step budget's default,
which graphs exist), not on the command line. Same idea and keys as the reference where it has them
(miniserve/engine/describe.py:22-67)."""

from __future__ import annotations

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


def _checkout_commit(root: Path) -> str | None:
    """The commit a checkout stands at, read from its ``.git`` folder (no git program needed); None
    where the tree is no checkout."""
    try:
        head = (root / ".git" / "HEAD").read_text().strip()
        if not head.startswith("ref:"):
            return head or None
        ref = head.split(None, 1)[1]
        loose = root / ".git" / ref
        if loose.is_file():
            return loose.read_text().strip() or None
        for line in (root / ".git" / "packed-refs").read_text().splitlines():
            if line.endswith(" " + ref):
                return line.split()[0]
    except OSError:
        pass
    return None


def runtime_description() -> dict:
    """What the engine stands on: the device as the HIP runtime describes it, the library versions, and
    which build of the kernel sources is loaded (its file name carries the digest of the sources, so it
    identifies the code even where the tree is a bare copy without history)."""
    import torch

    from ..kernels import build

    record = {"torch": torch.__version__, "hip": getattr(torch.version, "hip", None)}
    device = {"gpu": None, "gpu_arch": None, "gpu_memory_bytes": None, "compute_units": None, "l2_cache_bytes": None}
    if torch.cuda.is_available():
        p = torch.cuda.get_device_properties(0)
        device = {"gpu": p.name, "gpu_arch": getattr(p, "gcnArchName", None), "gpu_memory_bytes": p.total_memory,
                  "compute_units": p.multi_processor_count, "l2_cache_bytes": getattr(p, "L2_cache_size", None)}
    record.update(device)
    record["kernel_library"] = build.kernel_library_name()
    record["block_core_library"] = build.core_library_name()
    record["commit"] = _checkout_commit(Path(__file__).resolve().parents[2])
    return record
