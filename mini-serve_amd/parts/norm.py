"""RMSNorm: ``y = w * x * rsqrt(mean(x^2) + eps)``, statistics and scaling in float32, plain weight
(not ``1 + w``) as in the reference (miniserve/model/qwen3.py:78-82). The reference rounds to the
model dtype before the weight product; here the whole expression is evaluated in float32 and
rounded once, which is what its fused operators do (miniserve/model/fused.py:188-194)."""

from __future__ import annotations

from ..config.spec import PartSpec
from .base import Norm, TensorSpec
from .registry import register


@register("norm", "rmsnorm")
class RMSNorm(Norm):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.width = int(spec["width"])
        self.eps = float(spec["eps"])
        self.weight = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        return {spec["tensor"]: TensorSpec((int(spec["width"]),), init="ones")}

    def bind(self, tensors) -> None:
        self.weight = tensors[self.spec["tensor"]]

    def forward(self, x, rows=None, add=None):
        """``x``: float32 ``[T, width]``; ``rows``: optional int32 row indices to normalise (the
        others are skipped); ``add``: a pending sum added into the normalised rows of ``x`` first.
        Returns the compute dtype, ``[T or len(rows), width]``."""
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, self.rt.dtype, rows, add)

    def parameters_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()
