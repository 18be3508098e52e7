"""One step's batch as the kernels see it.

A step runs rows ``(request cache, next tokens, wanted places)``: portions of prompts beside
single decoded tokens, cut anywhere. ``StepBatch`` flattens them: ``token_ids``, ``positions`` and
``token_row`` per token, ``row_start`` offsets, and per cache group the block tables (dense
``[rows, width]``) and the slot of every new token. Everything is written into one pinned int32
staging buffer and uploaded with one copy (the reference uploads ids, positions, slots and the
packed tables separately, miniserve/engine/model_runner.py:232-260).
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..cache.pages import pack_tables


@dataclass
class StepRow:
    cache: object  # RequestCache
    tokens: list
    want: list  # indices into ``tokens`` whose logits are asked for
    # The row's last token is not known on the host yet: it is element ``feed`` of the device tensor
    # of sampled tokens that the step is given (``tokens[-1]`` is ignored). None: all tokens are known.
    feed: int | None = None


@dataclass
class GroupBatch:
    block_table: torch.Tensor  # int32 [rows, width]
    slots: torch.Tensor  # int32 [tokens]


class StepBatch:
    """Device-side description of a step. Built by ``BatchBuilder.build``. ``decode_tokens`` /
    ``prefill_tokens``: flat indices of the tokens of rows that bring one token / several tokens
    (None when all tokens are of one kind: the list is then the identity)."""

    __slots__ = (
        "num_rows", "num_tokens", "num_wanted", "token_ids", "positions", "token_row", "row_start", "starts",
        "kv_lens", "state_slots", "want_rows", "groups", "row_lens", "row_starts_host", "max_kv_len", "is_decode",
        "num_decode_tokens", "decode_tokens", "prefill_tokens", "_tiles", "memo", "feed",
    )

    def __init__(self):
        self._tiles = None
        # What parts derive from the step's tokens alone and share between layers (a rotation table,
        # say), by a key of the part's choosing. The model empties it at the start of every pass.
        self.memo = {}

    def prefill_tiles(self, tile_tokens: int):
        """Tiles of at most ``tile_tokens`` consecutive new tokens of the rows that bring several
        tokens: ``(first flat token index [n], token count [n], n)`` on the device, heaviest
        (deepest into its sequence) first. Built once per tile size and step."""
        cache = getattr(self, "_tiles", None)
        if cache is None:
            cache = self._tiles = {}
        if tile_tokens not in cache:
            from ..kernels.ops import build_prefill_tiles

            cache[tile_tokens] = build_prefill_tiles(self.row_lens, self.row_starts_host, tile_tokens, self.token_ids.device)
        return cache[tile_tokens]


def _align(n: int, to: int = 4) -> int:
    return -(-n // to) * to


class BatchBuilder:
    def __init__(self, device, num_groups: int):
        self.device = torch.device(device)
        self.num_groups = num_groups
        self._host = None
        self._dev = None
        self._fence = None

    def _reserve(self, n: int) -> None:
        if self._host is None or self._host.numel() < n:
            cap = max(4096, 1 << (n - 1).bit_length())
            if self._fence is not None:
                self._fence.synchronize()
            self._host = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._dev = torch.empty(cap, dtype=torch.int32, device=self.device)

    def build(self, rows: list[StepRow], starts: list[int]) -> StepBatch:
        """``starts[i]``: tokens row ``i`` held before this step (its tables already include the
        new tokens)."""
        B = len(rows)
        lens = [len(r.tokens) for r in rows]
        T = sum(lens)
        n_want = sum(len(r.want) for r in rows)
        # table rows are a multiple of 4 entries wide: kernels fetch the page ids of a key tile with one 16-byte load
        widths = [_align(max(1, max(r.cache.tables[g].num_entries for r in rows))) for g in range(self.num_groups)]

        seg = {}
        off = 0

        def take(name, n):
            nonlocal off
            seg[name] = (off, n)
            off += _align(n)

        take("ids", T); take("pos", T); take("row", T)
        take("row_start", B + 1); take("starts", B); take("kv_lens", B); take("state", B)
        take("want", n_want)
        fed = any(r.feed is not None for r in rows)
        if fed:
            take("feed", B)
        n_dec = sum(1 for n in lens if n == 1)
        mixed = 0 < n_dec < B
        if mixed:
            take("dec_tok", n_dec); take("pre_tok", T - n_dec)
        for g in range(self.num_groups):
            take(f"slots{g}", T)
            take(f"table{g}", B * widths[g])
        self._reserve(off)
        if self._fence is not None:
            self._fence.synchronize()  # the previous upload has read the staging buffer
        host = self._host.numpy()

        def view(name):
            o, n = seg[name]
            return host[o : o + n]

        ids, pos, row = view("ids"), view("pos"), view("row")
        want = view("want")
        t = w = 0
        row_start = view("row_start")
        for i, (r, s, n) in enumerate(zip(rows, starts, lens)):
            row_start[i] = t
            ids[t : t + n] = r.tokens
            pos[t : t + n] = np.arange(s, s + n, dtype=np.int32)
            row[t : t + n] = i
            for k in r.want:
                want[w] = t + k
                w += 1
            t += n
        row_start[B] = T
        if mixed:
            dec, pre = view("dec_tok"), view("pre_tok")
            t = d = q = 0
            for n in lens:
                if n == 1:
                    dec[d] = t
                    d += 1
                else:
                    pre[q : q + n] = np.arange(t, t + n, dtype=np.int32)
                    q += n
                t += n
        if fed:
            view("feed")[:] = [-1 if r.feed is None else r.feed for r in rows]
        view("starts")[:] = starts
        view("kv_lens")[:] = [s + n for s, n in zip(starts, lens)]
        view("state")[:] = [r.cache.state_slot if r.cache.state_slot is not None else 0 for r in rows]
        for g in range(self.num_groups):
            sl = view(f"slots{g}")
            t = 0
            for r, n in zip(rows, lens):
                r.cache.tables[g].tail_slots_into(n, sl[t : t + n])
                t += n
            pack_tables([r.cache.tables[g] for r in rows], view(f"table{g}").reshape(B, widths[g]))

        self._dev[:off].copy_(self._host[:off], non_blocking=True)
        if self._fence is None:
            self._fence = torch.cuda.Event()
        self._fence.record()

        def dview(name):
            o, n = seg[name]
            return self._dev[o : o + n]

        b = StepBatch()
        b.num_rows, b.num_tokens, b.num_wanted = B, T, n_want
        b.token_ids, b.positions, b.token_row = dview("ids"), dview("pos"), dview("row")
        b.row_start, b.starts, b.kv_lens, b.state_slots = dview("row_start"), dview("starts"), dview("kv_lens"), dview("state")
        b.want_rows = dview("want")
        b.feed = dview("feed") if fed else None
        b.groups = [GroupBatch(dview(f"table{g}").view(B, widths[g]), dview(f"slots{g}")) for g in range(self.num_groups)]
        b.row_lens = lens
        b.row_starts_host = list(starts)
        b.max_kv_len = max(s + n for s, n in zip(starts, lens))
        b.is_decode = n_dec == B
        b.num_decode_tokens = n_dec
        # None stands for the identity list (every token is one)
        b.decode_tokens = dview("dec_tok") if mixed else None
        b.prefill_tokens = dview("pre_tok") if mixed else None
        return b
