"""Captured HIP graphs for pure decode steps.

One graph per (batch bucket, table-width bucket): batch buckets are the powers of two below the
largest batch and the largest batch itself (miniserve/engine/cuda_graph.py:49-65); the width bucket is
the power of two that holds the longest block table of the step. A graph is captured the first
time its key is needed. Its inputs live in one static int32 device buffer with a fixed layout
(token ids, positions, slots, block tables, ...), filled from a pinned staging buffer by one copy
before each replay. Rows beyond the real batch are padding: token 0 at position 0, written to and
read from the pool's extra page, which no allocator hands out (:217-248).

The logits come back as a view of the graph's static output, valid until the next replay.
"""

from __future__ import annotations

import gc
import weakref

import numpy as np
import torch

from .batch import GroupBatch, StepBatch, _align


def graph_buckets(max_bs: int) -> list[int]:
    out, b = [], 1
    while b < max_bs:
        out.append(b)
        b *= 2
    return out + [max_bs]


class _Captured:
    __slots__ = ("graph", "host", "dev", "seg", "batch", "logits", "fence")


class DecodeGraphs:
    MIN_WIDTH = 16

    def __init__(self, runner, max_bs: int):
        # No cycle with the runner: the graphs must go when the runner goes, not whenever the cyclic
        # collector gets to them (which may be in the middle of another runner's capture).
        self.runner = weakref.proxy(runner)
        self.buckets = graph_buckets(max_bs)
        self.max_bs = max_bs
        self.captured: dict = {}
        self.pool = None
        self.latest = None  # the captured graph the latest ``run`` replayed
        self.num_groups = len(runner.layout.groups)

    def usable(self, rows) -> bool:
        return len(rows) <= self.max_bs and all(len(r.tokens) == 1 and list(r.want) == [0] for r in rows)

    def _key(self, rows):
        g = next(b for b in self.buckets if b >= len(rows))
        need = max(max(t.num_entries for t in r.cache.tables) for r in rows)
        w = self.MIN_WIDTH
        while w < need:
            w *= 2
        return g, w

    def _layout(self, g: int, w: int):
        seg, off = {}, 0
        for name, n in [("ids", g), ("pos", g), ("row", g), ("row_start", g + 1), ("starts", g), ("kv_lens", g),
                        ("state", g), ("want", g), ("feed", g)] + [
            item for k in range(self.num_groups) for item in ((f"slots{k}", g), (f"table{k}", g * w))
        ]:
            seg[name] = (off, n)
            off += _align(n)
        return seg, off

    def _capture(self, g: int, w: int) -> _Captured:
        c = _Captured()
        c.seg, total = self._layout(g, w)
        dev = self.runner.device
        c.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        c.dev = torch.zeros(total, dtype=torch.int32, device=dev)
        c.fence = torch.cuda.Event()
        h = c.host.numpy()

        def hv(name):
            o, n = c.seg[name]
            return h[o : o + n]

        def dv(name):
            o, n = c.seg[name]
            return c.dev[o : o + n]

        hv("row")[:] = np.arange(g)
        hv("row_start")[:] = np.arange(g + 1)
        hv("want")[:] = np.arange(g)
        self._fill_padding(c, 0, g, w)
        b = StepBatch()
        b.num_rows = b.num_tokens = b.num_wanted = g
        b.token_ids, b.positions, b.token_row = dv("ids"), dv("pos"), dv("row")
        b.row_start, b.starts, b.kv_lens, b.state_slots = dv("row_start"), dv("starts"), dv("kv_lens"), dv("state")
        b.want_rows = dv("want")
        b.feed = None  # tokens still on the device are put into the static buffer before the replay
        b.groups = [GroupBatch(dv(f"table{k}").view(g, w), dv(f"slots{k}")) for k in range(self.num_groups)]
        b.row_lens, b.row_starts_host, b.max_kv_len, b.is_decode = [1] * g, [0] * g, w * self.runner.page_size, True
        b.num_decode_tokens, b.decode_tokens, b.prefill_tokens = g, None, None
        c.batch = b
        c.dev.copy_(c.host)
        model, pool = self.runner.model, self.runner.pool
        # Warm up on a side stream (first launches load code objects), then capture.
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.forward(b, pool)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        c.graph = torch.cuda.CUDAGraph()
        # The cyclic collector stays off while the stream is capturing: what it might free then (a
        # graph, a stream, an event of some earlier object) may not be freed during a capture.
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(c.graph, pool=self.pool):
                c.logits = model.forward(b, pool)
        finally:
            if collecting:
                gc.enable()
        if self.pool is None:
            self.pool = c.graph.pool()
        return c

    def _fill_padding(self, c: _Captured, first: int, g: int, w: int) -> None:
        h = c.host.numpy()
        for name, val in (("ids", 0), ("pos", 0), ("starts", 0), ("kv_lens", 1), ("state", self.runner.max_running)):
            o, n = c.seg[name]
            h[o + first : o + g] = val
        for k in range(self.num_groups):
            dummy = self.runner.pool.dummy_page(k)
            o, _ = c.seg[f"slots{k}"]
            h[o + first : o + g] = dummy * self.runner.page_size
            o, _ = c.seg[f"table{k}"]
            h[o + first * w : o + g * w] = dummy

    def run(self, rows, starts, feed_from=None):
        """Replay the graph for these decode rows (their tables already hold the new token). Rows with
        ``feed`` take their token from the device tensor ``feed_from``."""
        from ..cache.pages import pack_tables

        g, w = key = self._key(rows)
        c = self.captured.get(key)
        if c is None:
            c = self.captured[key] = self._capture(g, w)
        B = len(rows)
        c.fence.synchronize()  # the previous upload has read the staging buffer
        h = c.host.numpy()

        def hv(name):
            o, n = c.seg[name]
            return h[o : o + n]

        hv("ids")[:B] = [r.tokens[0] for r in rows]
        fed = any(r.feed is not None for r in rows)
        if fed:
            hv("feed")[:B] = [-1 if r.feed is None else r.feed for r in rows]
            hv("feed")[B:] = -1
        hv("pos")[:B] = starts
        hv("starts")[:B] = starts
        hv("kv_lens")[:B] = [s + 1 for s in starts]
        hv("state")[:B] = [r.cache.state_slot if r.cache.state_slot is not None else 0 for r in rows]
        for k in range(self.num_groups):
            sl = hv(f"slots{k}")
            for i, r in enumerate(rows):
                r.cache.tables[k].tail_slots_into(1, sl[i : i + 1])
            dummy = self.runner.pool.dummy_page(k)
            pack_tables([r.cache.tables[k] for r in rows], hv(f"table{k}").reshape(g, w), pad_rows=g - B, pad_page=dummy)
        if B < g:
            self._fill_padding(c, B, g, w)
        c.dev.copy_(c.host, non_blocking=True)
        c.fence.record()
        if fed:
            o, n = c.seg["feed"]
            self.runner.model.rt.ops.feed_tokens(c.batch.token_ids, None, c.dev[o : o + n], feed_from)
        c.graph.replay()
        self.latest = c
        return c.logits[:B]
