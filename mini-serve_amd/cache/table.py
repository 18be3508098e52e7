"""Per-request map from token positions to pages (Python implementation).

Token ``pos`` lives in page ``blocks[pos // block_size]`` at offset ``pos % block_size``
(miniserve/cache/block_table.py:19-89). Beyond the reference: ``release_before(pos)`` gives back
the whole pages that lie entirely before ``pos`` (a window has passed them); their entries become
``NO_BLOCK`` and are never read again.
"""

from __future__ import annotations

from collections.abc import Sequence

NO_BLOCK = -1


class BlockTable:
    def __init__(self, allocator, prefix_blocks: Sequence[int] = ()):
        self.allocator = allocator
        self.block_size = allocator.block_size
        if len(set(prefix_blocks)) != len(prefix_blocks):
            raise ValueError(f"duplicate block in prefix {list(prefix_blocks)}")
        allocator.incref(prefix_blocks)
        self.blocks: list[int] = list(prefix_blocks)
        self.num_tokens = len(self.blocks) * self.block_size
        self.first_live = 0  # index of the first entry that still holds a page

    @property
    def num_blocks(self) -> int:
        """Entries of the table (pages held plus entries already given back)."""
        return len(self.blocks)

    @property
    def num_held(self) -> int:
        return len(self.blocks) - self.first_live

    @property
    def capacity(self) -> int:
        return len(self.blocks) * self.block_size

    @property
    def last_block_len(self) -> int:
        if self.num_tokens == 0:
            return 0
        return self.num_tokens - (len(self.blocks) - 1) * self.block_size

    def blocks_needed(self, n: int) -> int:
        if n < 0:
            raise ValueError(f"cannot append {n} tokens")
        return max(0, -(-(self.num_tokens + n) // self.block_size) - len(self.blocks))

    def append_tokens(self, n: int) -> list[int]:
        new = self.allocator.allocate(self.blocks_needed(n))
        self.blocks += new
        self.num_tokens += n
        return new

    def slot(self, pos: int) -> int:
        if not 0 <= pos < self.num_tokens:
            raise IndexError(f"position {pos} out of range [0, {self.num_tokens})")
        b = self.blocks[pos // self.block_size]
        if b == NO_BLOCK:
            raise IndexError(f"position {pos} lies in a page that was given back")
        return b * self.block_size + pos % self.block_size

    def tail_slots(self, n: int) -> list[int]:
        if not 0 <= n <= self.num_tokens:
            raise IndexError(f"tail of {n} tokens out of range [0, {self.num_tokens}]")
        bs = self.block_size
        start = self.num_tokens - n
        if n and start // bs < self.first_live:
            raise IndexError(f"position {start} lies in a page that was given back")
        return [self.blocks[p // bs] * bs + p % bs for p in range(start, self.num_tokens)]

    def tail_slots_into(self, n: int, out) -> None:
        """``tail_slots(n)`` written into the int32 array ``out`` (its first ``n`` entries)."""
        out[:n] = self.tail_slots(n)

    def rewind(self, n: int) -> None:
        if not 0 <= n <= self.num_tokens:
            raise IndexError(f"cannot rewind {n} of {self.num_tokens} tokens")
        if (self.num_tokens - n) // self.block_size < self.first_live and n:
            raise IndexError("cannot rewind into pages that were given back")
        self.num_tokens -= n

    def release_before(self, pos: int) -> int:
        """Give back every page whose tokens all lie before ``pos``. Returns how many."""
        upto = min(max(pos, 0) // self.block_size, len(self.blocks))
        if upto <= self.first_live:
            return 0
        gone = self.blocks[self.first_live : upto]
        self.allocator.free(gone)
        for i in range(self.first_live, upto):
            self.blocks[i] = NO_BLOCK
        self.first_live = upto
        return len(gone)

    def release(self) -> None:
        self.allocator.free(self.blocks[self.first_live :])
        self.blocks = []
        self.num_tokens = 0
        self.first_live = 0


def pack_tables(tables, out, pad_rows: int = 0, pad_block: int = 0) -> int:
    """Write the tables as rows of a dense int32 matrix ``out[rows, width]`` (numpy view of a
    reusable pinned buffer): row ``i`` holds table ``i``'s entries, the rest of the row is
    ``pad_block``; ``pad_rows`` further rows hold ``pad_block`` alone. One call per batch
    (the reference packs its CSR layout the same way, miniserve/cache/block_table.py:92-113).
    Returns the number of entries written from tables."""
    rows = len(tables) + pad_rows
    if pad_rows < 0:
        raise ValueError("pad_rows must be >= 0")
    if tables and not isinstance(tables[0], BlockTable):
        from .native import pack_native

        if out.ndim != 2 or not out.flags.c_contiguous:
            raise ValueError("packing buffer must be a contiguous matrix")
        return pack_native(tables, out, pad_rows, pad_block)
    if out.ndim != 2 or out.shape[0] < rows:
        raise ValueError(f"packing buffer too small: need {rows} rows, got {out.shape}")
    width = out.shape[1]
    total = 0
    for i, t in enumerate(tables):
        n = len(t.blocks)
        if n > width:
            raise ValueError(f"packing buffer too narrow: table of {n} entries, width {width}")
        out[i, :n] = t.blocks
        out[i, n:] = pad_block
        total += n
    out[len(tables) : rows, :] = pad_block
    return total
