"""The cache manager: pages for keys and values, a block table per request and group, and slots
for fixed-size per-request state.

Cache slots of the model's run order are sorted into *groups* by what they keep per token
(KV heads, head size, all keys or a window of them). Each group has pages and an allocator of its
own, and every request holds one block table per group. Pages go back to their group when the
request ends, is preempted, or (windowed groups) when the window has passed them, and are handed
out again, newest first.

The reference has one uniform pool over all layers and one table per request
(miniserve/cache/kv_pool.py:32-44, miniserve/cache/kv_cache.py:33-136); its request-level calls
``acquire / abandon / release / reserve / num_available`` are kept in meaning, without the radix
tree: prefixes are not shared between requests (the table's shared-prefix constructor is there
for it).
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .pages import OutOfBlocks, PageAllocator
from .state import StateSlots


@dataclass(frozen=True)
class CacheGroup:
    """Cache slots that keep the same planes per token over the same window (0: every token)."""

    index: int
    planes: tuple  # of parts.base.CachePlane: name, heads, width, token_minor
    window: int
    slots: tuple[int, ...]

    @property
    def elements_per_token(self) -> int:
        return sum(p.heads * p.width for p in self.planes)


@dataclass(frozen=True)
class StateGroup:
    """The fixed-size state of one cache slot: named tensors, each with a shape per request and a dtype."""

    slot: int
    tensors: tuple  # of parts.base.StateTensor


@dataclass(frozen=True)
class CacheLayout:
    groups: tuple[CacheGroup, ...]
    states: tuple[StateGroup, ...]
    group_of_slot: dict = field(default_factory=dict, compare=False)

    @classmethod
    def from_needs(cls, needs) -> "CacheLayout":
        """``needs``: ``CacheSlotNeed`` list of a model (``DecoderModel.cache_slots()``)."""
        by_key: dict[tuple, list[int]] = {}
        planes_of: dict[tuple, tuple] = {}
        states = []
        for n in needs:
            if n.kv is not None:
                key = (tuple((p.name, p.heads, p.width, p.token_minor) for p in n.kv.planes), n.kv.window)
                by_key.setdefault(key, []).append(n.slot)
                planes_of[key] = tuple(n.kv.planes)
            if n.state is not None:
                states.append(StateGroup(n.slot, tuple(n.state.tensors)))
        groups = tuple(
            CacheGroup(i, planes_of[key], key[1], tuple(slots)) for i, (key, slots) in enumerate(sorted(by_key.items()))
        )
        return cls(groups, tuple(states), {s: g.index for g in groups for s in g.slots})

    def bytes_per_page(self, page_size: int, itemsize: int) -> list[int]:
        return [len(g.slots) * page_size * g.elements_per_token * itemsize for g in self.groups]


class RequestCache:
    """What one live request holds: a table per group, a state slot, and how many tokens are in."""

    __slots__ = ("tables", "state_slot", "num_tokens")

    def __init__(self, tables, state_slot):
        self.tables = tables
        self.state_slot = state_slot
        self.num_tokens = 0

    @property
    def num_blocks(self) -> int:
        return sum(t.num_held for t in self.tables)


class CacheManager:
    def __init__(
        self,
        layout: CacheLayout,
        page_size: int,
        pages_per_group: list[int],
        num_state_slots: int,
        max_step_tokens: int | None = None,
        allocator_class=PageAllocator,
    ):
        if len(pages_per_group) != len(layout.groups):
            raise ValueError("one page count per group is needed")
        self.layout = layout
        self.page_size = page_size
        self.max_step_tokens = max_step_tokens
        self.allocators = [allocator_class(n, page_size) for n in pages_per_group]
        self.state_slots = StateSlots(num_state_slots)
        self.live: set[int] = set()  # ids of RequestCache objects handed out

    # ------------------------------------------------------------------ sizes

    @property
    def num_groups(self) -> int:
        return len(self.allocators)

    def pages(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def free_pages(self) -> list[int]:
        return [a.num_free for a in self.allocators]

    def total_pages(self) -> list[int]:
        return [a.num_pages for a in self.allocators]

    def peak_pages(self, total_tokens: int, step_tokens: int | None = None) -> list[int]:
        """Most pages per group a request holds at any time on its way to ``total_tokens``, fed in
        steps of at most ``step_tokens`` tokens. A windowed group needs the window plus one step."""
        step = step_tokens if step_tokens else self.max_step_tokens
        out = []
        for g in self.layout.groups:
            full = self.pages(total_tokens)
            if g.window and step:
                full = min(full, self.pages(g.window - 1 + step) + 1)
            out.append(full)
        return out

    def fits_alone(self, total_tokens: int, step_tokens: int | None = None) -> bool:
        """Whether a request of ``total_tokens``, fed in steps of at most ``step_tokens``, could run with
        the whole pool to itself."""
        return all(p <= t for p, t in zip(self.peak_pages(total_tokens, step_tokens), self.total_pages()))

    # ------------------------------------------------------------------ request life

    def acquire(self) -> RequestCache:
        """A fresh handle: empty tables and a state slot. Takes no pages."""
        slot = self.state_slots.acquire()
        rc = RequestCache([a.new_table() for a in self.allocators], slot)
        self.live.add(id(rc))
        return rc

    def pages_needed(self, rc: RequestCache, n: int) -> list[int]:
        """Pages each group must hand out to append ``n`` tokens to ``rc`` now."""
        return [t.pages_needed(n) for t in rc.tables]

    def outstanding(self, rc: RequestCache, total_tokens: int, step_tokens: int | None = None) -> list[int]:
        """Pages per group ``rc`` may still draw (net of what it gives back) until it holds
        ``total_tokens`` tokens, fed in steps of at most ``step_tokens``."""
        peak = self.peak_pages(total_tokens, step_tokens)
        out = []
        for g, t, p in zip(self.layout.groups, rc.tables, peak):
            held = t.num_held
            if g.window:
                out.append(max(0, p - held))
            else:
                out.append(max(0, p - t.num_entries))
        return out

    def can_extend(self, rc: RequestCache, n: int) -> bool:
        return all(need <= a.num_free for need, a in zip(self.pages_needed(rc, n), self.allocators))

    def extend(self, rc: RequestCache, n: int) -> None:
        """Make room for ``n`` more tokens in every group, all or nothing: on ``OutOfBlocks`` no
        table has changed (miniserve/engine/model_runner.py:309-315)."""
        self._check_live(rc)
        need = self.pages_needed(rc, n)
        for g, (k, a) in enumerate(zip(need, self.allocators)):
            if k > a.num_free:
                raise OutOfBlocks(f"group {g}: need {k} free pages, {a.num_free} free")
        for t in rc.tables:
            t.append(n)
        rc.num_tokens += n

    def advance(self, rc: RequestCache) -> int:
        """After a step: give back the pages of windowed groups that no later query can see
        (a query at position p >= num_tokens sees keys from p - window + 1 on). Returns how many."""
        freed = 0
        for g, t in zip(self.layout.groups, rc.tables):
            if g.window:
                freed += t.release_before(rc.num_tokens - g.window + 1)
        return freed

    def release(self, rc: RequestCache) -> None:
        """End of the request (finished, aborted or preempted): every page and the state slot go back."""
        self._check_live(rc)
        for t in rc.tables:
            t.release()
        self.state_slots.release(rc.state_slot)
        rc.state_slot = None
        rc.num_tokens = 0
        self.live.discard(id(rc))

    # ------------------------------------------------------------------ checks

    def _check_live(self, rc: RequestCache) -> None:
        if id(rc) not in self.live:
            raise RuntimeError("this cache handle was released or never acquired here")

    @property
    def idle(self) -> bool:
        return all(a.num_free == a.num_pages for a in self.allocators) and (
            self.state_slots.num_free == self.state_slots.num_slots
        )

    def check_invariants(self) -> None:
        for a in self.allocators:
            a.check_invariants()
        self.state_slots.check_invariants()
