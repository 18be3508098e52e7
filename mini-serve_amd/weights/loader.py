"""Weights from a model folder, by tensor name.

Every ``*.safetensors`` file of the folder is read (sorted, every key) as the reference does
(miniserve/model/weights.py:104-114); names and shapes are checked against what the model's parts
declare, and one ``ValueError`` lists missing tensors, unexpected tensors and wrong shapes, so a
wrong or partial checkpoint fails at load and never inside a forward pass (:121-133).

Dtypes: with compute dtype bfloat16, 16-bit float tensors are kept in bfloat16 and a tensor stored
in 32-bit stays 32-bit (the part that owns it then computes with it in 32-bit); with compute
dtype float32 every float tensor is widened to float32 (exact). Integer tables become int32.
A part may read a tensor under a second name (``Part.aliases``: a tied head reads the embedding's
table as its own weight, :116-119,135-136): nothing is stored for that name, a duplicate in the file is
dropped, and the name maps to the source's tensor itself.
"""

from __future__ import annotations

from pathlib import Path

import torch
from safetensors import safe_open

from ..config.spec import ModelSpec
from ..parts.model import expected_aliases, expected_tensors

_FLOAT16 = (torch.bfloat16, torch.float16)
MAX_LISTED = 8


class WeightsError(ValueError):
    """The checkpoint does not match the model: carries the three lists."""

    def __init__(self, path, missing, unexpected, mismatched):
        self.missing, self.unexpected, self.mismatched = missing, unexpected, mismatched

        def show(items):
            more = f" (+{len(items) - MAX_LISTED} more)" if len(items) > MAX_LISTED else ""
            return f"{items[:MAX_LISTED]}{more}"

        super().__init__(
            f"checkpoint {path} does not match its config: missing={show(missing)} "
            f"unexpected={show(unexpected)} shape_mismatch={show(mismatched)}"
        )


def _place(t: torch.Tensor, kind: str, dtype: torch.dtype) -> torch.Tensor:
    if kind == "int":
        if t.dtype.is_floating_point:
            raise TypeError("a float tensor where an integer table is expected")
        return t.to(torch.int32)
    if not t.dtype.is_floating_point:
        raise TypeError("an integer tensor where a float tensor is expected")
    if dtype == torch.float32:
        return t.to(torch.float32)
    if t.dtype in _FLOAT16:
        return t.to(torch.bfloat16)
    return t.to(torch.float32)  # stored in 32-bit (or wider): stays 32-bit


def load_weights(
    path: str | Path,
    spec: ModelSpec,
    dtype: torch.dtype = torch.bfloat16,
    device: str | torch.device = "cuda",
) -> dict[str, torch.Tensor]:
    if dtype not in (torch.float32, torch.bfloat16):
        raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
    path = Path(path)
    files = sorted(path.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors files in {path}")
    want = expected_tensors(spec)
    aliases = expected_aliases(spec)  # names the parts read another tensor under: nothing is stored for them

    weights: dict[str, torch.Tensor] = {}
    unexpected: list[str] = []
    mismatched: list[str] = []
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as sf:
            for name in sf.keys():
                if name in aliases:
                    continue  # the source tensor wins over a stored duplicate
                ts = want.get(name)
                if ts is None:
                    unexpected.append(name)
                    continue
                shape = tuple(sf.get_slice(name).get_shape())
                if shape != ts.shape:
                    mismatched.append(f"{name}: {shape} != {ts.shape}")
                    continue
                try:
                    weights[name] = _place(sf.get_tensor(name), ts.kind, dtype).to(device).contiguous()
                except TypeError as e:
                    mismatched.append(f"{name}: {e}")
    missing = sorted(want.keys() - weights.keys() - {m.split(":")[0] for m in mismatched})
    if missing or unexpected or mismatched:
        raise WeightsError(path, missing, sorted(unexpected), sorted(mismatched))
    for name, source in aliases.items():
        weights[name] = weights[source]
    return weights
