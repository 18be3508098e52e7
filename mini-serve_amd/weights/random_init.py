"""Random weights from a configuration and a seed, in memory or as a model folder
(``config.json`` + ``model.safetensors``) that the by-name loader reads back.

The reference has no such mode; its tests alone build random tensors from the expected shapes
and save them as a checkpoint (tests/test_weights.py:26-32). Tensors are drawn in sorted name
order from one seeded generator, each by the rule its part declares (``TensorSpec.init``): ``normal``
N(0, std) for matrices and embeddings, ``ones`` for norm weights (all one, or uniform in
``norm_range``), ``uniform`` U(-std, std), ``zeros``; integer tables uniformly from ``[0, high)``.
Float values are rounded to bfloat16 before they are stored, so the float32 and the bfloat16 path
start from the same numbers.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

import torch
from safetensors.torch import save_file

from ..config.registry import config_from_dict
from ..config.spec import ModelSpec
from ..parts.model import expected_tensors


@dataclass(frozen=True)
class Init:
    std: float = 0.02
    norm_range: tuple[float, float] | None = None  # None: norm weights are 1.0


def random_tensors(
    spec: ModelSpec,
    seed: int,
    init: Init = Init(),
    dtype: torch.dtype = torch.bfloat16,
    device: str | torch.device = "cpu",
) -> dict[str, torch.Tensor]:
    """Name -> tensor for every tensor the model's parts declare, each drawn by its own ``init``
    rule. Drawing happens on ``device`` (a GPU generator draws other numbers than the CPU's; a
    folder written once is what fixes the values)."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    f32 = dict(dtype=torch.float32, device=device)
    out = {}
    for name, ts in sorted(expected_tensors(spec).items()):
        if ts.kind == "int":
            out[name] = torch.randint(0, ts.high, ts.shape, generator=gen, dtype=torch.int32, device=device)
            continue
        if ts.init == "ones":
            if init.norm_range is None:
                t = torch.ones(ts.shape, **f32)
            else:
                lo, hi = init.norm_range
                t = torch.rand(ts.shape, generator=gen, **f32) * (hi - lo) + lo
        elif ts.init == "zeros":
            t = torch.zeros(ts.shape, **f32)
        elif ts.init == "uniform":
            t = (torch.rand(ts.shape, generator=gen, **f32) * 2 - 1) * init.std
        else:
            t = torch.randn(ts.shape, generator=gen, **f32) * init.std
        out[name] = t.to(torch.bfloat16).to(dtype)
    return out


def write_model_folder(
    path: str | Path,
    config: dict,
    seed: int,
    init: Init = Init(),
    store_dtype: torch.dtype = torch.bfloat16,
) -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a config.json dictionary)."""
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    spec = config_from_dict(config).to_spec()
    tensors = random_tensors(spec, seed, init, dtype=store_dtype)
    (path / "config.json").write_text(json.dumps(config, indent=1))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return path


def main(argv=None) -> int:
    import argparse

    from ..config.presets import PRESETS, preset

    ap = argparse.ArgumentParser(description="write a model folder with random weights")
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--preset", choices=sorted(PRESETS))
    src.add_argument("--config", help="a config.json to take the sizes from")
    ap.add_argument("--out", required=True)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--std", type=float, default=0.02)
    ap.add_argument("--norm-range", type=float, nargs=2, default=None, metavar=("LO", "HI"))
    ap.add_argument("--store-dtype", choices=("bfloat16", "float32"), default="bfloat16")
    a = ap.parse_args(argv)
    cfg = preset(a.preset) if a.preset else json.loads(Path(a.config).read_text())
    init = Init(a.std, tuple(a.norm_range) if a.norm_range else None)
    write_model_folder(a.out, cfg, a.seed, init, getattr(torch, a.store_dtype))
    print(a.out)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
