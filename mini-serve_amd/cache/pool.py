"""Device storage of the cache: per group one tensor of pages, per stateful slot one tensor of
state slots.

Pages of a group: ``[slots_in_group, 2 (K, V), pages + 1, kv_heads, page_size * head_dim]`` in the
compute dtype, zero-initialised. One KV head of one page is a contiguous run, so an attention
workgroup that owns a KV head streams whole runs. Keys lie ``[page_size, head_dim]`` inside the run;
values lie transposed, ``[head_dim, page_size]``: the tokens of one head element are contiguous,
which is the order the matrix cores need them in for the probability-value product. (The reference keeps ``[2, layers, blocks, block_size, kv_heads,
head_dim]``, miniserve/cache/kv_pool.py:32-44.) The one extra page past the allocator's range is
the dummy page that padding rows of a captured decode graph write to and read from
(miniserve/engine/model_runner.py:111-113).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .manager import CacheLayout


@dataclass
class LayerCache:
    """What a mixer gets for one run-order entry."""

    k: torch.Tensor  # [pages + 1, kv_heads, page_size, head_dim]
    v: torch.Tensor  # [pages + 1, kv_heads, head_dim, page_size]
    block_table: torch.Tensor  # int32 [rows, width] page ids of this group
    slots: torch.Tensor  # int32 [tokens] page * page_size + offset of each new token
    writes: bool
    page_size: int
    window: int


class KVPool:
    def __init__(self, layout: CacheLayout, page_size: int, pages_per_group: list[int], num_state_slots: int, dtype, device):
        self.layout = layout
        self.page_size = page_size
        self.dtype = dtype
        self.device = torch.device(device)
        self.pages_per_group = list(pages_per_group)
        self.buffers = [
            torch.zeros((len(g.slots), 2, n + 1, g.num_kv_heads, page_size, g.head_dim), dtype=dtype, device=device)
            for g, n in zip(layout.groups, pages_per_group)
        ]
        self._where = {s: (g.index, i) for g in layout.groups for i, s in enumerate(g.slots)}
        self.states = {
            s.slot: torch.zeros((num_state_slots + 1, *s.shape), dtype=getattr(torch, s.dtype), device=device)
            for s in layout.states
        }

    @property
    def num_bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self.buffers)

    def dummy_page(self, group: int) -> int:
        return self.pages_per_group[group]

    def bytes_per_token(self) -> int:
        """Cache bytes one token occupies over all groups (windows not counted)."""
        item = torch.empty((), dtype=self.dtype).element_size()
        return sum(2 * len(g.slots) * g.num_kv_heads * g.head_dim * item for g in self.layout.groups)

    def view(self, slot: int, batch, writes: bool) -> LayerCache | None:
        where = self._where.get(slot)
        if where is None:
            return None
        gi, i = where
        gb = batch.groups[gi]
        buf = self.buffers[gi]
        g = self.layout.groups[gi]
        v = buf[i, 1].view(buf.shape[2], g.num_kv_heads, g.head_dim, self.page_size)
        return LayerCache(buf[i, 0], v, gb.block_table, gb.slots, writes, self.page_size, g.window)

    def state_view(self, slot: int, batch):
        return self.states.get(slot)
