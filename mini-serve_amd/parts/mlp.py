"""Gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases
(miniserve/model/qwen3.py:128-131). Gate and up are one matrix product over one weight that holds
both (the reference concatenates them, miniserve/model/fused.py:41,195; here their rows alternate in
runs of 16 where the width allows, so that a matrix kernel's lane holds gate and up of the same output
and can finish the activation itself); the activation product is evaluated in float32 and rounded
once; the down projection adds into the residual stream in its epilogue."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import FeedForward, TensorSpec
from .registry import register

@register("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.prefix = spec.get("prefix", "")
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = spec.get("activation", "silu")
        if self.activation not in rt.ops.ACTIVATIONS:
            raise NotImplementedError(f"activation {self.activation!r} is not supported, expected one of {sorted(rt.ops.ACTIVATIONS)}")
        self.gate_up = self.down = None
        self.block = 0  # rows per run of gate / up rows in gate_up (0: all gates, then all ups)

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
        ops = self.rt.ops
        self.block = ops.GATE_BLOCK if self.inter % ops.GATE_BLOCK == 0 else 0
        self.gate_up = ops.interleave_gate_up(g, u) if self.block else torch.cat((g, u), dim=0).contiguous()
        self.down = tensors[p + "down_proj.weight"]

    def forward(self, x, residual):
        ops = self.rt.ops
        m = ops.gated_linear(x, self.gate_up, self.activation, out_dtype=self.rt.dtype, block=self.block)
        return ops.linear(m, self.down, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.gate_up, self.down))

    def flops(self, rows) -> int:
        return 2 * sum(n for n, _ in rows) * 3 * self.hidden * self.inter
