"""Block arrangements: where the norms and the residual sums sit around a mixer and a
feed-forward. ``prenorm`` is the reference's (miniserve/model/qwen3.py:212-216):
``h += mixer(norm(h)); h += feed_forward(norm(h))``."""

from __future__ import annotations

from ..config.spec import PartSpec
from .base import Block, TensorSpec
from .registry import part_class, register


@register("block", "prenorm")
class PreNormBlock(Block):
    def __init__(self, spec: PartSpec, rt, mixer, feed_forward):
        super().__init__(spec, rt, mixer, feed_forward)
        mn, fn = spec["mixer_norm"], spec["ffn_norm"]
        self.mixer_norm = part_class("norm", mn)(mn, rt)
        self.ffn_norm = part_class("norm", fn)(fn, rt)

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        out = {}
        for key in ("mixer_norm", "ffn_norm"):
            s = spec[key]
            out.update(part_class("norm", s).tensors(s))
        return out

    def bind(self, tensors) -> None:
        self.mixer_norm.bind(tensors)
        self.ffn_norm.bind(tensors)

    def forward(self, residual, batch, cache, state, pending=None):
        x = self.mixer_norm.forward(residual, add=pending)
        pending = self.mixer.forward(x, batch, cache, state, residual)
        y = self.ffn_norm.forward(residual, add=pending)
        return self.feed_forward.forward(y, residual)

    def parameters_bytes(self) -> int:
        return self.mixer_norm.parameters_bytes() + self.ffn_norm.parameters_bytes()
