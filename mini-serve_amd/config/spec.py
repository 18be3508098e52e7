"""Architecture-neutral description of a decoder: which parts, with which constants, in which order.

A typed configuration (one per architecture, e.g. ``Qwen3Config``) reads the architecture's own
``config.json`` keys and lowers itself to a ``ModelSpec``. Everything below the configuration
(weights, parts, cache, step function) sees only the ``ModelSpec``: no part knows which model it
is in, and no size or constant lives in code.

The reference hard-codes one layer shape in one class (miniserve/model/qwen3.py:110-131,212-216);
this description is the seam that lets layers differ and be arranged as data.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from types import MappingProxyType
from typing import Any, Mapping


def _freeze(params: Mapping[str, Any]) -> Mapping[str, Any]:
    return MappingProxyType(dict(params))


@dataclass(frozen=True)
class PartSpec:
    """One part: a registry ``kind`` and the sizes / constants it is built with."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self):
        object.__setattr__(self, "params", _freeze(self.params))

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One set of layer weights: a block arrangement around a mixer and a feed-forward.

    ``prefix`` is the tensor-name prefix of the layer in the checkpoint (``model.layers.3.``).
    ``block`` names the arrangement (where norms and residual sums sit) and carries the norms.
    """

    prefix: str
    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order: run ``layer``'s weights over cache slot ``cache``.

    A layer may appear in several entries (its weights are run twice); then each entry normally
    names a cache slot of its own. ``writes_cache=False`` lets an entry read the slot another
    entry wrote instead of keeping keys and values of its own.
    """

    layer: int
    cache: int | None
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    run_order: tuple[RunEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    max_position: int | None = None

    def __post_init__(self):
        slots_written: set[int] = set()
        for e in self.run_order:
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run order names layer {e.layer}, the model has {len(self.layers)}")
            if e.cache is None:
                continue
            if e.writes_cache:
                if e.cache in slots_written:
                    raise ValueError(f"cache slot {e.cache} is written by two run entries")
                slots_written.add(e.cache)
            elif e.cache not in slots_written:
                raise ValueError(f"run entry reads cache slot {e.cache} before any entry wrote it")

    @property
    def num_cache_slots(self) -> int:
        used = [e.cache for e in self.run_order if e.cache is not None]
        return max(used) + 1 if used else 0
