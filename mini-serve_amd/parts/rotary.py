"""Rotary position encoding, rotate-half pairing (j, j + dim/2) over the first ``dim`` elements of
each head. Frequencies ``inv_freq[j] = 1 / theta**(2j/dim)`` are computed on the host in float32
exactly as the reference does (miniserve/model/qwen3.py:97-100) and moved once; the angles
``float32(position) * inv_freq[j]`` and their cosines and sines are formed in float32 on the device
once per step, as a table that every layer with the same frequencies shares (the reference builds
float32 tables per pass, :105-108)."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import PositionEncoding, Rotation
from .registry import register


@register("position", "rotary")
class Rotary(PositionEncoding):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.dim = int(spec["dim"])
        self.theta = float(spec["theta"])
        if self.dim < 2 or self.dim % 2:
            raise ValueError(f"rotary dim {self.dim} must be even")
        expo = torch.arange(0, self.dim, 2, dtype=torch.int64).to(torch.float32) / self.dim
        self.inv_freq_host = 1.0 / (self.theta**expo)
        self.inv_freq = self.inv_freq_host.to(rt.device) if rt is not None else None

    def rotation(self, batch) -> Rotation:
        key = ("rotary", self.dim, self.theta)
        table = batch.memo.get(key)
        if table is None:
            table = batch.memo[key] = self.rt.ops.rope_table(batch.positions, self.inv_freq)
        return Rotation(self.dim, table)


@register("position", "none")
class NoPosition(PositionEncoding):
    """No position signal inside the mixer."""
