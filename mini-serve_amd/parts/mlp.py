"""Gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases
(miniserve/model/qwen3.py:128-131). Gate and up are one matrix product over row-concatenated
weights ``[gate; up]`` (miniserve/model/fused.py:41,195); the activation product is evaluated in
float32 and rounded once; the down projection adds into the residual stream in its epilogue."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import FeedForward, TensorSpec
from .registry import register

ACTIVATIONS = ("silu",)


@register("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.prefix = spec.get("prefix", "")
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = spec.get("activation", "silu")
        if self.activation not in ACTIVATIONS:
            raise NotImplementedError(f"activation {self.activation!r} is not supported, expected {ACTIVATIONS}")
        self.gate_up = self.down = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        p = spec.get("prefix", "")
        h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
        return {
            p + "gate_proj.weight": TensorSpec((i, h)),
            p + "up_proj.weight": TensorSpec((i, h)),
            p + "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, tensors) -> None:
        p = self.prefix
        g, u = tensors[p + "gate_proj.weight"], tensors[p + "up_proj.weight"]
        if g.dtype != u.dtype:
            raise ValueError(f"{p}gate/up projections are stored in different dtypes")
        self.gate_up = torch.cat((g, u), dim=0).contiguous()
        self.down = tensors[p + "down_proj.weight"]

    def forward(self, x, residual):
        ops = self.rt.ops
        gu = ops.linear(x, self.gate_up, out_dtype=self.rt.dtype, defer=True)
        m = ops.act_mul(gu, self.activation, out_dtype=self.rt.dtype)
        return ops.linear(m, self.down, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.gate_up, self.down))
