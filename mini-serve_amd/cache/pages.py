"""Pages of one layer group and the per-request tables over them (Python implementation).

A group's bookkeeping is three int32 arrays, the layout the C++ core keeps too: ``holders[page]`` (0 =
free), and a stack of free page ids of which the top is handed out next. A request's table is a
growing int32 array of page ids; token ``pos`` lives in page ``entries[pos // page_size]`` at offset
``pos % page_size``. Slots of new tokens and the packed tables of a batch are computed by array
arithmetic straight into the pinned staging buffer a step uploads.

The order in which pages are handed out is a contract (the C++ core and the reference's vectors
are checked id for id, miniserve/cache/block_allocator.py:24-107, block_table.py:19-89): a fresh
group hands out 0, 1, 2, ...; pages given back are used again newest first; taking pages is all or
nothing; giving back checks the whole call before anything changes. Beyond the reference: a table
gives back the pages a window has passed (``release_before``); those entries read ``NO_PAGE``.
"""

from __future__ import annotations

from collections.abc import Iterable

import numpy as np

NO_PAGE = -1


class OutOfBlocks(RuntimeError):
    """A group has fewer free pages than were asked for; nothing was taken."""


def _ids(pages) -> np.ndarray:
    return np.asarray(pages if isinstance(pages, np.ndarray) else list(pages), dtype=np.int32).reshape(-1)


class PageAllocator:
    backend = "python"

    def __init__(self, num_pages: int, page_size: int):
        if num_pages < 1 or page_size < 1:
            raise ValueError(f"a group needs at least one page of at least one token, got {num_pages} x {page_size}")
        self.num_pages = num_pages
        self.page_size = page_size
        self.holders = np.zeros(num_pages, dtype=np.int32)
        self.stack = np.arange(num_pages - 1, -1, -1, dtype=np.int32)  # stack[:top] are free, stack[top - 1] goes first
        self.top = num_pages

    # -------------------------------------------------------------- counts

    @property
    def num_free(self) -> int:
        return self.top

    @property
    def num_used(self) -> int:
        return self.num_pages - self.top

    def holders_of(self, page: int) -> int:
        self._in_range(_ids([page]))
        return int(self.holders[page])

    # -------------------------------------------------------------- pages in and out

    def take(self, n: int) -> list[int]:
        """``n`` free pages, each with one holder: the caller."""
        if n < 0:
            raise ValueError(f"cannot take {n} pages")
        if n > self.top:
            raise OutOfBlocks(f"{n} pages wanted, {self.top} of {self.num_pages} free")
        got = self.stack[self.top - n : self.top][::-1]
        self.top -= n
        self.holders[got] = 1
        return got.tolist()

    def hold(self, pages: Iterable[int]) -> None:
        """One more holder for each of ``pages`` (a second table shares them). Free pages cannot be shared."""
        ids = _ids(pages)
        self._in_range(ids)
        if ids.size and (self.holders[ids] == 0).any():
            raise ValueError(f"page {int(ids[self.holders[ids] == 0][0])} is free and cannot be shared")
        np.add.at(self.holders, ids, 1)

    def give_back(self, pages: Iterable[int]) -> None:
        """One holder of each of ``pages`` lets go (a page may be named once per holder). A page whose
        last holder left is free again and the next to be handed out."""
        ids = _ids(pages)
        self._in_range(ids)
        named, times = np.unique(ids, return_counts=True)
        short = self.holders[named] < times
        if short.any():
            p = int(named[short][0])
            raise ValueError(f"page {p} is given back {int(times[short][0])} times but has {int(self.holders[p])} holders")
        if named.size == ids.size:  # the usual call: every page once
            self.holders[ids] -= 1
            freed = ids[self.holders[ids] == 0]
        else:  # a page goes free where its last holder is named
            freed = []
            for p in ids.tolist():
                self.holders[p] -= 1
                if self.holders[p] == 0:
                    freed.append(p)
            freed = np.asarray(freed, dtype=np.int32)
        self.stack[self.top : self.top + freed.size] = freed
        self.top += int(freed.size)

    def new_table(self, shared: Iterable[int] = ()) -> "PageTable":
        return PageTable(self, shared)

    # -------------------------------------------------------------- checks

    def _in_range(self, ids: np.ndarray) -> None:
        if ids.size and (int(ids.min()) < 0 or int(ids.max()) >= self.num_pages):
            bad = int(ids[(ids < 0) | (ids >= self.num_pages)][0])
            raise IndexError(f"page {bad} does not exist: the group has pages 0..{self.num_pages - 1}")

    def check_invariants(self) -> None:
        free = self.stack[: self.top]
        assert np.unique(free).size == free.size, "a page lies twice on the free stack"
        assert (self.holders >= 0).all(), "a page has a negative number of holders"
        is_free = np.zeros(self.num_pages, dtype=bool)
        is_free[free] = True
        assert (is_free == (self.holders == 0)).all(), "the free stack and the holder counts disagree"


class PageTable:
    """One request's pages in one group, in the order of its tokens."""

    def __init__(self, allocator: PageAllocator, shared: Iterable[int] = ()):
        shared = _ids(shared)
        if np.unique(shared).size != shared.size:
            raise ValueError(f"duplicate page in the shared prefix {shared.tolist()}")
        allocator.hold(shared)
        self.allocator = allocator
        self.page_size = allocator.page_size
        self._entries = np.empty(max(8, int(shared.size)), dtype=np.int32)
        self._entries[: shared.size] = shared
        self.num_entries = int(shared.size)  # pages held plus entries already given back
        self.first_live = 0  # index of the first entry that still holds a page
        self.num_tokens = self.num_entries * self.page_size  # a shared prefix is whole pages

    # -------------------------------------------------------------- views

    @property
    def entries(self) -> np.ndarray:
        return self._entries[: self.num_entries]

    @property
    def pages(self) -> list[int]:
        return self.entries.tolist()

    @property
    def num_held(self) -> int:
        return self.num_entries - self.first_live

    # -------------------------------------------------------------- growth

    def pages_needed(self, n: int) -> int:
        """Pages the group must hand out before ``n`` more tokens fit."""
        if n < 0:
            raise ValueError(f"cannot append {n} tokens")
        return max(0, -(-(self.num_tokens + n) // self.page_size) - self.num_entries)

    def append(self, n: int) -> list[int]:
        """Room for ``n`` more tokens; returns the pages newly taken (all or nothing)."""
        new = self.allocator.take(self.pages_needed(n))
        if new:
            end = self.num_entries + len(new)
            if end > self._entries.size:
                grown = np.empty(max(end, 2 * self._entries.size), dtype=np.int32)
                grown[: self.num_entries] = self.entries
                self._entries = grown
            self._entries[self.num_entries : end] = new
            self.num_entries = end
        self.num_tokens += n
        return new

    def rewind(self, n: int) -> None:
        """Forget the last ``n`` tokens but keep their pages: recomputed tokens land in the same slots."""
        if not 0 <= n <= self.num_tokens:
            raise IndexError(f"cannot rewind {n} of {self.num_tokens} tokens")
        if n and (self.num_tokens - n) // self.page_size < self.first_live:
            raise IndexError("cannot rewind into pages that were given back")
        self.num_tokens -= n

    # -------------------------------------------------------------- where tokens live

    def slot(self, pos: int) -> int:
        if not 0 <= pos < self.num_tokens:
            raise IndexError(f"position {pos} out of range [0, {self.num_tokens})")
        page = int(self._entries[pos // self.page_size])
        if page == NO_PAGE:
            raise IndexError(f"position {pos} lies in a page that was given back")
        return page * self.page_size + pos % self.page_size

    def tail_slots_into(self, n: int, out: np.ndarray) -> None:
        """Slots of the last ``n`` tokens, written into the first ``n`` entries of ``out`` (int32)."""
        if not 0 <= n <= self.num_tokens:
            raise IndexError(f"tail of {n} tokens out of range [0, {self.num_tokens}]")
        if n == 0:
            return
        first = self.num_tokens - n
        if n == 1 and first // self.page_size >= self.first_live:  # a decode step: no array arithmetic for one token
            out[0] = int(self._entries[first // self.page_size]) * self.page_size + first % self.page_size
            return
        if first // self.page_size < self.first_live:
            raise IndexError(f"position {first} lies in a page that was given back")
        pos = np.arange(first, self.num_tokens, dtype=np.int32)
        out[:n] = self._entries[pos // self.page_size] * self.page_size + pos % self.page_size

    def tail_slots(self, n: int) -> list[int]:
        out = np.empty(max(n, 0), dtype=np.int32)
        self.tail_slots_into(n, out)
        return out.tolist()

    # -------------------------------------------------------------- pages going back

    def release_before(self, pos: int) -> int:
        """Give back every page whose tokens all lie before ``pos``. Returns how many."""
        upto = min(max(pos, 0) // self.page_size, self.num_entries)
        if upto <= self.first_live:
            return 0
        self.allocator.give_back(self._entries[self.first_live : upto])
        self._entries[self.first_live : upto] = NO_PAGE
        gone = upto - self.first_live
        self.first_live = upto
        return gone

    def release(self) -> None:
        self.allocator.give_back(self._entries[self.first_live : self.num_entries])
        self.num_entries = self.num_tokens = self.first_live = 0


def pack_tables(tables, out: np.ndarray, pad_rows: int = 0, pad_page: int = 0) -> int:
    """The tables of a batch as rows of the dense int32 matrix ``out[rows, width]`` (a view of the
    step's staging buffer): row ``i`` holds table ``i``'s entries and then ``pad_page``; ``pad_rows``
    further rows hold ``pad_page`` alone. One call per batch and group (the reference packs a CSR
    layout the same way, miniserve/cache/block_table.py:92-113). Returns the entries written from tables."""
    if pad_rows < 0:
        raise ValueError("pad_rows must be >= 0")
    if out.ndim != 2 or not out.flags.c_contiguous:
        raise ValueError("the packing buffer must be a contiguous matrix")
    if tables and not isinstance(tables[0], PageTable):
        from .native import pack_native

        return pack_native(tables, out, pad_rows, pad_page)
    rows = len(tables) + pad_rows
    if out.shape[0] < rows:
        raise ValueError(f"the packing buffer has {out.shape[0]} rows, {rows} are needed")
    out[:rows] = pad_page
    total = 0
    for i, t in enumerate(tables):
        if t.num_entries > out.shape[1]:
            raise ValueError(f"the packing buffer is {out.shape[1]} entries wide, a table has {t.num_entries}")
        out[i, : t.num_entries] = t.entries
        total += t.num_entries
    return total
