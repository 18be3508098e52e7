"""Grouped-query softmax attention over the paged cache.

Per layer, in the reference's order (miniserve/model/qwen3.py:110-126): q/k/v projections without
bias, per-head RMSNorm of q and k (one ``[head_dim]`` weight each, shared by all heads), rotation
of q and k, store of k and v into the cache, causal attention in which query head ``h`` reads KV
head ``h // (heads / kv_heads)`` with ``scale`` on the scores, output projection. Here the three
projections are one matrix product over row-concatenated weights (as the reference's fused path
does, miniserve/model/fused.py:204-206); norm, rotation and cache store are one kernel (in a step of
single tokens they are part of the attention kernel); the output
projection adds into the residual stream in its epilogue, or (few rows) leaves partial sums pending
for the next norm to add.

``window > 0`` restricts a query at position p to keys p-window+1 .. p (no counterpart in the
reference). ``qk_norm_eps=None`` switches the per-head norms off; ``position`` may be ``none``.
"""

from __future__ import annotations

import warnings

import torch

from ..config.spec import PartSpec
from .base import KVNeed, Mixer, TensorSpec
from .registry import part_class, register


@register("mixer", "gqa_attention")
class GQAttention(Mixer):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.prefix = spec.get("prefix", "")
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.scale = float(spec["scale"])
        self.qk_norm_eps = spec.get("qk_norm_eps")
        self.window = int(spec.get("window") or 0)
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} query heads are no multiple of {self.kv_heads} KV heads")
        # What the attention kernels refuse is refused here, when the model is built, not in its first step.
        if self.head_dim % 16 or not 16 <= self.head_dim <= 256:
            raise ValueError(f"head_dim {self.head_dim} is not supported: the attention kernels take multiples of 16 from 16 to 256")
        if not self.scale > 0:
            raise ValueError(f"the attention scale must be positive, not {self.scale}")
        if rt is not None and rt.dtype == torch.bfloat16 and not (
                self.head_dim in (64, 128) and self.heads // self.kv_heads <= 16):
            warnings.warn(
                f"attention with head_dim {self.head_dim} and {self.heads // self.kv_heads} query heads per KV head runs the "
                "generic kernel in bfloat16 (one wave per token and head): the matrix-core kernels take head sizes 64 and 128 "
                "with up to 16 query heads per KV head", stacklevel=2)
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos)(pos, rt)
        self.qkv = self.o = self.q_norm = self.k_norm = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        p = spec.get("prefix", "")
        h, d = int(spec["hidden_size"]), int(spec["head_dim"])
        hq, hkv = int(spec["num_heads"]), int(spec["num_kv_heads"])
        out = {
            p + "q_proj.weight": TensorSpec((hq * d, h)),
            p + "k_proj.weight": TensorSpec((hkv * d, h)),
            p + "v_proj.weight": TensorSpec((hkv * d, h)),
            p + "o_proj.weight": TensorSpec((h, hq * d)),
        }
        if spec.get("qk_norm_eps") is not None:
            out[p + "q_norm.weight"] = TensorSpec((d,), init="ones")
            out[p + "k_norm.weight"] = TensorSpec((d,), init="ones")
        return out

    def bind(self, tensors) -> None:
        p = self.prefix
        parts = [tensors[p + n + "_proj.weight"] for n in ("q", "k", "v")]
        if len({t.dtype for t in parts}) != 1:
            raise ValueError(f"{p}q/k/v projections are stored in different dtypes")
        self.qkv = torch.cat(parts, dim=0).contiguous()
        self.o = tensors[p + "o_proj.weight"]
        if self.qk_norm_eps is not None:
            self.q_norm = tensors[p + "q_norm.weight"]
            self.k_norm = tensors[p + "k_norm.weight"]

    def kv_need(self) -> KVNeed:
        return KVNeed.keys_values(self.kv_heads, self.head_dim, self.window)

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        qkv = ops.linear(x, self.qkv, out_dtype=self.rt.dtype, defer=True)
        rot = self.position.rotation(batch)
        table = rot.table if rot is not None else None
        pairing = rot.pairing if rot is not None else "halves"
        if ops.decode_attention_fusable(qkv, batch, self.q_norm, self.k_norm, table, cache.k, cache.v,
                                        self.heads, self.kv_heads, self.head_dim, pairing):
            # a step of single tokens: norm, rotation, cache store and attention are one kernel
            # ... and, with few rows, the reduction of the key splits and the output projection another
            out = ops.decode_attention_fused(
                qkv, self.q_norm, self.k_norm, 0.0 if self.qk_norm_eps is None else float(self.qk_norm_eps), table,
                cache.writes, cache.k, cache.v, cache.block_table, batch, self.heads, self.kv_heads, self.head_dim,
                self.scale, self.window, project=self.o if self.o.dtype == torch.bfloat16 else None,
            )
            if isinstance(out, ops.SplitSum):
                return out  # the projection's partial sums: pending, for the next reader of the stream
            return ops.linear(out, self.o, accumulate_into=residual, defer=True)
        q = ops.qk_norm_rope_store(
            qkv, cache.slots if cache.writes else None,
            self.q_norm, self.k_norm, 0.0 if self.qk_norm_eps is None else float(self.qk_norm_eps),
            table,
            cache.k, cache.v, self.heads, self.kv_heads, self.head_dim, out_dtype=self.rt.dtype, pairing=pairing,
        )
        out = ops.paged_attention(
            q, cache.k, cache.v, cache.block_table, batch, self.heads, self.kv_heads, self.head_dim,
            self.scale, self.window,
        )
        return ops.linear(out, self.o, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        ts = [self.qkv, self.o] + ([self.q_norm, self.k_norm] if self.q_norm is not None else [])
        return sum(t.numel() * t.element_size() for t in ts)

    def flops(self, rows) -> int:
        """The four projections, and both attention products over every (query, visible key) pair: a query
        at position p sees keys ``max(0, p - window + 1) .. p``."""
        tokens = sum(n for n, _ in rows)
        pairs = 0
        for n, cached in rows:
            for p in (range(cached, cached + n) if self.window else ()):
                pairs += min(p + 1, self.window)
            if not self.window:
                pairs += n * cached + n * (n + 1) // 2
        width = self.heads * self.head_dim
        linear = 2 * tokens * self.hidden * (width + 2 * self.kv_heads * self.head_dim) + 2 * tokens * width * self.hidden
        return linear + 4 * pairs * width
