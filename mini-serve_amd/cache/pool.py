"""Device storage of the cache: per group and plane one tensor of pages, per stateful slot its state tensors.

A group's mixers say what they keep per token as a list of planes (``parts.base.CachePlane``); the pool
builds one tensor per plane, ``[slots_in_group, pages + 1, heads, page_size, width]`` in the compute
dtype, zero-initialised, or, for a ``token_minor`` plane, ``[slots_in_group, pages + 1, heads, width,
page_size]``. One head of one page is a contiguous run, so an attention workgroup that owns a KV head
streams whole runs. The attention mixer keeps two planes: keys ``[page_size, head_dim]`` inside the run
and values transposed, ``[head_dim, page_size]``: the tokens of one head element are contiguous, which
is the order the matrix cores need them in for the probability-value product. (The reference keeps
``[2, layers, blocks, block_size, kv_heads, head_dim]``, miniserve/cache/kv_pool.py:32-44.) The one
extra page past the allocator's range is the dummy page that padding rows of a captured decode graph
write to and read from (miniserve/engine/model_runner.py:111-113).

State: per cache slot that asked for it, one tensor ``[state_slots + 1, *shape]`` per named state
tensor, each in its own dtype; the extra row belongs to padding rows.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .manager import CacheLayout


@dataclass
class LayerCache:
    """What a mixer gets for one run-order entry: its planes' page tensors by name (leading dimension
    pages + 1), the block tables of the step's rows and the slot of every new token."""

    planes: dict  # name -> [pages + 1, heads, page_size, width] or, token_minor, [pages + 1, heads, width, page_size]
    block_table: torch.Tensor  # int32 [rows, width] page ids of this group
    slots: torch.Tensor  # int32 [tokens] page * page_size + offset of each new token
    writes: bool
    page_size: int
    window: int

    @property
    def k(self) -> torch.Tensor:
        return self.planes["k"]

    @property
    def v(self) -> torch.Tensor:
        return self.planes["v"]


class KVPool:
    def __init__(self, layout: CacheLayout, page_size: int, pages_per_group: list[int], num_state_slots: int, dtype, device):
        self.layout = layout
        self.page_size = page_size
        self.dtype = dtype
        self.device = torch.device(device)
        self.pages_per_group = list(pages_per_group)
        self.buffers = [
            {
                p.name: torch.zeros(
                    (len(g.slots), n + 1, p.heads) + ((p.width, page_size) if p.token_minor else (page_size, p.width)),
                    dtype=dtype, device=device)
                for p in g.planes
            }
            for g, n in zip(layout.groups, pages_per_group)
        ]
        self._where = {s: (g.index, i) for g in layout.groups for i, s in enumerate(g.slots)}
        self.states = {
            s.slot: {t.name: torch.zeros((num_state_slots + 1, *t.shape), dtype=getattr(torch, t.dtype), device=device)
                     for t in s.tensors}
            for s in layout.states
        }

    @property
    def num_bytes(self) -> int:
        return sum(b.numel() * b.element_size() for planes in self.buffers for b in planes.values())

    def dummy_page(self, group: int) -> int:
        return self.pages_per_group[group]

    def bytes_per_token(self) -> int:
        """Cache bytes one token occupies over all groups (windows not counted)."""
        item = torch.empty((), dtype=self.dtype).element_size()
        return sum(len(g.slots) * g.elements_per_token * item for g in self.layout.groups)

    def view(self, slot: int, batch, writes: bool) -> LayerCache | None:
        where = self._where.get(slot)
        if where is None:
            return None
        gi, i = where
        gb = batch.groups[gi]
        planes = {name: buf[i] for name, buf in self.buffers[gi].items()}
        return LayerCache(planes, gb.block_table, gb.slots, writes, self.page_size, self.layout.groups[gi].window)

    def state_view(self, slot: int, batch) -> dict | None:
        """The state tensors of a cache slot by name (None if its mixer keeps none); row
        ``batch.state_slots[b]`` of each is request ``b``'s."""
        return self.states.get(slot)
