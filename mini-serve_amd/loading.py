"""From a model folder to a model on the GPU: the three calls every entry point makes, in the
reference's manner (``Qwen3Config.from_dict(load_config(p))``, ``load_weights(p)``, model class;
miniserve/server/__main__.py:73-75, bench/offline.py:395-413), with the class chosen by
``config.json``'s architecture name."""

from __future__ import annotations

from pathlib import Path

import torch

from .config.registry import config_from_dict, load_config_dict
from .parts.base import Runtime
from .parts.model import DecoderModel
from .weights.loader import load_weights
from .weights.random_init import Init, random_tensors

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return DTYPES[name]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}, expected one of {sorted(DTYPES)}") from None


def runtime(dtype, device="cuda:0") -> Runtime:
    from .kernels import ops

    ops.library()  # fails loudly here if the kernels are missing
    return Runtime(parse_dtype(dtype), torch.device(device), ops)


def load_model(path: str | Path, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    cfg = config_from_dict(load_config_dict(path))
    spec = cfg.to_spec()
    rt = runtime(dtype, device)
    weights = load_weights(path, spec, rt.dtype, rt.device)
    model = DecoderModel(spec, weights, rt)
    model.config = cfg
    return model


def random_model(config: dict, seed: int = 0, dtype="bfloat16", device="cuda:0", init: Init = Init()) -> DecoderModel:
    """A model with random weights drawn on the device (no folder is written)."""
    cfg = config_from_dict(config)
    spec = cfg.to_spec()
    rt = runtime(dtype, device)
    weights = random_tensors(spec, seed, init, dtype=rt.dtype, device=rt.device)
    model = DecoderModel(spec, weights, rt)
    model.config = cfg
    return model
