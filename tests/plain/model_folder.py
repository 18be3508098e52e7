"""Reading a model folder (config.json + *.safetensors) with numpy alone.

The safetensors container is: 8 bytes little-endian header length, a JSON header mapping each
tensor name to ``{"dtype", "shape", "data_offsets"}``, then the raw little-endian data. The
reference reads the same files through the safetensors package (miniserve/model/weights.py:104-114).
"""

from __future__ import annotations

import json
import struct
from pathlib import Path

import numpy as np


def _bf16_to_f32(raw: np.ndarray) -> np.ndarray:
    # bfloat16 is the upper half of a float32.
    return (raw.astype(np.uint32) << 16).view(np.float32)


def read_safetensors(path: str | Path) -> dict[str, np.ndarray]:
    data = Path(path).read_bytes()
    (n,) = struct.unpack("<Q", data[:8])
    header = json.loads(data[8 : 8 + n])
    body = memoryview(data)[8 + n :]
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        shape = tuple(meta["shape"])
        dt = meta["dtype"]
        if dt == "BF16":
            arr = _bf16_to_f32(np.frombuffer(body[lo:hi], dtype="<u2"))
        elif dt == "F16":
            arr = np.frombuffer(body[lo:hi], dtype="<f2").astype(np.float32)
        elif dt == "F32":
            arr = np.frombuffer(body[lo:hi], dtype="<f4")
        elif dt == "F64":
            arr = np.frombuffer(body[lo:hi], dtype="<f8")
        elif dt == "I32":
            arr = np.frombuffer(body[lo:hi], dtype="<i4")
        elif dt == "I64":
            arr = np.frombuffer(body[lo:hi], dtype="<i8")
        else:
            raise ValueError(f"{name}: dtype {dt} not handled")
        out[name] = arr.reshape(shape)
    return out


def read_model_folder(path: str | Path) -> tuple[dict, dict[str, np.ndarray]]:
    """``(config dict, name -> float64 array)`` of every tensor in the folder."""
    path = Path(path)
    cfg = json.loads((path / "config.json").read_text())
    weights: dict[str, np.ndarray] = {}
    for f in sorted(path.glob("*.safetensors")):
        for k, v in read_safetensors(f).items():
            weights[k] = v.astype(np.float64) if v.dtype.kind == "f" else v
    if cfg.get("tie_word_embeddings", False):
        # The embedding wins over a duplicate lm_head (miniserve/model/weights.py:116-119,135-136).
        weights["lm_head.weight"] = weights["model.embed_tokens.weight"]
    return cfg, weights
