"""The generic decoder: parts assembled from a ``ModelSpec`` and run in the order it lists.

One class serves every registered architecture; an architecture is its typed configuration's
``to_spec``. The model owns no cache: the step function hands it a batch and the pool's views.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..config.spec import ModelSpec
from .base import KVNeed, Runtime, StateNeed, TensorSpec
from .registry import part_class


def expected_tensors(spec: ModelSpec) -> dict[str, TensorSpec]:
    """Every checkpoint tensor of the model with its shape, collected from the parts' own
    declarations (the reference lists them in one flat function, miniserve/model/weights.py:60-91)."""
    out: dict[str, TensorSpec] = {}

    def add(tensors: dict[str, TensorSpec], prefix: str = "") -> None:
        for name, ts in tensors.items():
            full = prefix + name
            if full in out and out[full] != ts:
                raise ValueError(f"tensor {full} is declared twice with different shapes")
            out[full] = ts

    add(part_class("embedding", spec.embedding).tensors(spec.embedding))
    for layer in spec.layers:
        add(part_class("block", layer.block).tensors(layer.block), layer.prefix)
        add(part_class("mixer", layer.mixer).tensors(layer.mixer), layer.prefix)
        add(part_class("feed_forward", layer.feed_forward).tensors(layer.feed_forward), layer.prefix)
    add(part_class("norm", spec.final_norm).tensors(spec.final_norm))
    add(part_class("head", spec.head).tensors(spec.head))
    return out


def expected_aliases(spec: ModelSpec) -> dict[str, str]:
    """Every tensor name a part reads under which nothing is stored, with the full name of the tensor
    that stands for it, collected from the parts' own ``aliases``. A source must be a declared tensor."""
    out: dict[str, str] = {}

    def add(aliases: dict[str, str], prefix: str = "") -> None:
        for name, source in aliases.items():
            out[prefix + name] = source

    add(part_class("embedding", spec.embedding).aliases(spec.embedding))
    for layer in spec.layers:
        for category, part in (("block", layer.block), ("mixer", layer.mixer), ("feed_forward", layer.feed_forward)):
            add(part_class(category, part).aliases(part), layer.prefix)
    add(part_class("norm", spec.final_norm).aliases(spec.final_norm))
    add(part_class("head", spec.head).aliases(spec.head))
    declared = expected_tensors(spec)
    for name, source in out.items():
        if name in declared:
            raise ValueError(f"tensor {name} is declared as stored and as an alias of {source}")
        if source not in declared:
            raise ValueError(f"tensor {name} is an alias of {source}, which no part declares")
    return out


@dataclass(frozen=True)
class CacheSlotNeed:
    """What one cache slot of the run order holds: paged keys/values and/or fixed-size state."""

    slot: int
    kv: KVNeed | None
    state: StateNeed | None


class DecoderModel:
    def __init__(self, spec: ModelSpec, weights: dict, rt: Runtime):
        self.spec = spec
        self.rt = rt
        self.dtype = rt.dtype
        self.device = rt.device
        self.vocab_size = spec.vocab_size

        weights = dict(weights)
        for name, source in expected_aliases(spec).items():
            weights[name] = weights[source]  # the same tensor under its second name

        def local(prefix: str, part_type, part_spec) -> dict:
            names = list(part_type.tensors(part_spec)) + list(part_type.aliases(part_spec))
            return {n: weights[prefix + n] for n in names}

        self.embedding = part_class("embedding", spec.embedding)(spec.embedding, rt)
        self.embedding.bind(weights)
        self.blocks = []
        for layer in spec.layers:
            mixer = part_class("mixer", layer.mixer)(layer.mixer, rt)
            mixer.bind(local(layer.prefix, type(mixer), layer.mixer))
            ffn = part_class("feed_forward", layer.feed_forward)(layer.feed_forward, rt)
            ffn.bind(local(layer.prefix, type(ffn), layer.feed_forward))
            block = part_class("block", layer.block)(layer.block, rt, mixer, ffn)
            block.bind(local(layer.prefix, type(block), layer.block))
            self.blocks.append(block)
        self.final_norm = part_class("norm", spec.final_norm)(spec.final_norm, rt)
        self.final_norm.bind(weights)
        self.head = part_class("head", spec.head)(spec.head, rt)
        self.head.bind(weights)

    # ------------------------------------------------------------------ cache needs

    def cache_slots(self) -> list[CacheSlotNeed]:
        """One entry per cache slot of the run order, from the mixer that writes it."""
        needs: dict[int, CacheSlotNeed] = {}
        for e in self.spec.run_order:
            if e.cache is None:
                continue
            mixer = self.blocks[e.layer].mixer
            need = CacheSlotNeed(e.cache, mixer.kv_need(), mixer.state_need())
            if e.writes_cache:
                needs[e.cache] = need
            elif (needs[e.cache].kv, needs[e.cache].state) != (need.kv, need.state):
                raise ValueError(
                    f"layer {e.layer} reads cache slot {e.cache} but needs {need}, the slot holds {needs[e.cache]}"
                )
        return [needs[s] for s in sorted(needs)]

    # ------------------------------------------------------------------ forward

    def forward(self, batch, pool):
        """Run the batch's tokens through every run-order entry and return float32 logits
        ``[len(batch.want_rows), vocab]`` at the wanted flat token indices."""
        with self.rt.ops.stream_scope():
            return self._forward(batch, pool)

    def _forward(self, batch, pool):
        batch.memo = {}  # what parts share between layers is made anew in every pass (a captured pass records it)
        residual = self.embedding.forward(batch.token_ids)
        pending = None  # a sum a layer left to be added to the residual stream by its next reader
        for e in self.spec.run_order:
            cache = pool.view(e.cache, batch, e.writes_cache) if e.cache is not None else None
            state = pool.state_view(e.cache, batch) if e.cache is not None else None
            pending = self.blocks[e.layer].forward(residual, batch, cache, state, pending)
        if batch.num_wanted == 0:
            return None
        x = self.final_norm.forward(residual, rows=batch.want_rows, add=pending)
        return self.head.forward(x)

    def step_flops(self, rows) -> int:
        """Floating-point operations of one step over ``rows`` (``(new tokens, cached tokens)`` per request),
        logits at one position per request: the sum of what the parts say of themselves."""
        total = self.final_norm.flops(rows) + self.head.flops(rows)
        for e in self.spec.run_order:
            b = self.blocks[e.layer]
            total += b.flops(rows) + b.mixer.flops(rows) + b.feed_forward.flops(rows)
        return total

    def decode_read_bytes(self) -> int:
        """Bytes of weights one decode step reads: every run-order entry's layer once, the final
        norm and the head (embedding rows are only gathered)."""
        total = self.final_norm.parameters_bytes() + self.head.parameters_bytes()
        for e in self.spec.run_order:
            b = self.blocks[e.layer]
            total += b.parameters_bytes() + b.mixer.parameters_bytes() + b.feed_forward.parameters_bytes()
        return total
