"""Token embedding and output head.

Embedding: ``h = E[token_ids]`` without scaling (miniserve/model/qwen3.py:211), widened to the
float32 residual stream. Head: ``logits = x W^T`` without bias, scaling or soft-cap
(miniserve/model/qwen3.py:152,186,195), returned in float32; a tied head reads the embedding's
tensor itself, no copy (miniserve/model/weights.py:116-119,135-136)."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import Embedding, Head, TensorSpec
from .registry import register


@register("embedding", "token_embedding")
class TokenEmbedding(Embedding):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.vocab = int(spec["vocab_size"])
        self.width = int(spec["width"])
        self.table = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        return {spec["tensor"]: TensorSpec((int(spec["vocab_size"]), int(spec["width"])))}

    def bind(self, tensors) -> None:
        self.table = tensors[self.spec["tensor"]]

    def forward(self, token_ids):
        return self.rt.ops.embed(token_ids, self.table)

    def parameters_bytes(self) -> int:
        return 0  # a decode step gathers single rows


@register("head", "linear_head")
class LinearHead(Head):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.vocab = int(spec["vocab_size"])
        self.width = int(spec["width"])
        self.tied_to = spec.get("tied_to")
        self.weight = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        if spec.get("tied_to"):
            return {}
        return {spec["tensor"]: TensorSpec((int(spec["vocab_size"]), int(spec["width"])))}

    @classmethod
    def aliases(cls, spec: PartSpec) -> dict[str, str]:
        return {spec["tensor"]: spec["tied_to"]} if spec.get("tied_to") else {}

    def bind(self, tensors) -> None:
        self.weight = tensors[self.spec["tensor"]]

    def forward(self, x):
        return self.rt.ops.linear(x, self.weight, out_dtype=torch.float32)

    def parameters_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def flops(self, rows) -> int:
        return 2 * len(rows) * self.vocab * self.width  # one wanted position per request
