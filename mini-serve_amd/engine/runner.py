"""The model runner: owns the model, the cache manager and the pool, and offers the one step
function every caller goes through (the scheduler's engine loop, trace replay, the benchmark).

``step(rows)`` runs only the tokens it is given, as one batch, from the cache that earlier steps
left, and returns float32 logits at the wanted places. It generalises the reference's
``ModelRunner.forward`` (last new token of every row, miniserve/engine/model_runner.py:220-261) and
``forward_tokens`` (every new position, :279-307).
"""

from __future__ import annotations

import torch

from ..cache.pages import OutOfBlocks
from ..cache.manager import CacheLayout, CacheManager, RequestCache
from ..cache.pool import KVPool
from ..parts.model import DecoderModel
from .batch import BatchBuilder, StepRow

MAX_STEP_TOKENS = 65535  # what one launch of the kernels takes (``kernels.ops.MAX_STEP_TOKENS``)

DEFAULT_PAGE_SIZE = 16


class ModelRunner:
    def __init__(
        self,
        model: DecoderModel,
        page_size: int = DEFAULT_PAGE_SIZE,
        kv_pool_tokens: int | None = None,
        kv_mem_fraction: float = 0.9,
        max_running: int = 64,
        max_step_tokens: int | None = None,
        allocator_class=None,
        decode_graph: bool = False,
        decode_graph_max_bs: int | None = None,
        request_step_tokens: int | None = None,
    ):
        """``kv_pool_tokens``: exact pool size in tokens (rounded down to whole pages; an error if
        it holds no page or does not fit, never clipped; miniserve/engine/model_runner.py:99-108);
        default: ``kv_mem_fraction`` of the memory that is free beyond the measured peak of the largest step
        (``kv_profile`` holds the figures).
        ``max_step_tokens``: most tokens one step carries (what the default pool size is measured with).
        ``request_step_tokens``: most tokens of one request in a step (the portion size of a chunked
        prefill; None: unbounded). With it a group that keeps a window holds at most the window and one
        step per running request, and gets only that many pages; the pool size given or measured is
        that of the groups that keep every token."""
        self.model = model
        self.device = model.device
        self.page_size = page_size
        self.max_running = max_running
        self.layout = CacheLayout.from_needs(model.cache_slots())
        self.allocator_class = allocator_class
        item = torch.empty((), dtype=model.dtype).element_size()
        group_bytes = self.layout.bytes_per_page(page_size, item)
        per_page = sum(group_bytes)
        step_tokens = min(max_step_tokens or 8192, MAX_STEP_TOKENS)
        graph_rows = (decode_graph_max_bs or max_running) if decode_graph else 0
        # What a windowed group needs at most: per running request the window, one step, and a page's slack.
        self.window_pages = [
            max_running * (-(-(g.window - 1 + request_step_tokens) // page_size) + 1) if g.window and request_step_tokens else None
            for g in self.layout.groups
        ]
        self.kv_profile = {"page_size": page_size, "bytes_per_page": per_page, "kv_mem_fraction": kv_mem_fraction}
        self.max_step_tokens_limit = MAX_STEP_TOKENS
        if kv_pool_tokens is not None:
            pages = kv_pool_tokens // page_size
            if pages < 1:
                raise ValueError(f"kv_pool_tokens={kv_pool_tokens} holds no page of {page_size} tokens")
            per_group = [pages if w is None else min(pages, w) for w in self.window_pages]
            if self.device.type == "cuda":
                free, _ = torch.cuda.mem_get_info(self.device)
                need = sum(n * b for n, b in zip(per_group, group_bytes))
                if need > free:
                    raise ValueError(
                        f"kv_pool_tokens={kv_pool_tokens} does not fit in memory: it needs {per_group} pages of {group_bytes} "
                        f"bytes per group, {free} bytes are free"
                    )
        else:
            if per_page == 0:
                pages, per_group = 1, [1 for _ in self.layout.groups]  # no mixer keeps anything per token: the pool is a formality
            elif self.device.type != "cuda":
                raise RuntimeError("the default pool size is measured on the GPU: give kv_pool_tokens")
            else:
                self.kv_profile.update(self._profile(step_tokens, max_running, graph_rows, kv_mem_fraction, group_bytes))
                pages, per_group = self.kv_profile["max_pages"], self.kv_profile["pages_per_group"]
                # a step larger than the one whose peak was measured could run out of memory beside the pool
                self.max_step_tokens_limit = step_tokens
        self.num_pages = pages
        self.pages_per_group = per_group
        self.cache = CacheManager(self.layout, page_size, per_group, max_running, max_step_tokens, **self._allocator_kw())
        self.pool = KVPool(self.layout, page_size, per_group, max_running, model.dtype, self.device)
        self.kv_profile.update(num_pages=pages, pages_per_group=list(per_group), kv_pool_tokens=pages * page_size,
                               pool_bytes=self.pool.num_bytes)
        self.builder = BatchBuilder(self.device, len(self.layout.groups))
        self.graphs = None
        if decode_graph and self.device.type == "cuda":
            from .graphs import DecodeGraphs

            self.graphs = DecodeGraphs(self, decode_graph_max_bs or max_running)
        self.steps = 0
        self.graph_steps = 0
        self._last = None  # the latest step's batch (or captured graph), for ``repeat_last_step``

    def _allocator_kw(self) -> dict:
        return {} if self.allocator_class is None else {"allocator_class": self.allocator_class}

    def split_bytes(self, budget: int, group_bytes: list[int]) -> tuple[int, list[int]]:
        """Pages per group that ``budget`` bytes buy: every group that keeps all tokens gets the same count
        (returned first), a windowed group its own need (``window_pages``) or that count, whichever is less."""
        fixed = [False] * len(group_bytes)
        while True:
            spent = sum(w * b for w, b, f in zip(self.window_pages, group_bytes, fixed) if f)
            rest = sum(b for b, f in zip(group_bytes, fixed) if not f)
            pages = (budget - spent) // rest if rest else 0
            more = [w is not None and not f and w < pages for w, f in zip(self.window_pages, fixed)]
            if not any(more):
                break
            fixed = [f or m for f, m in zip(fixed, more)]
        if not rest:  # every group keeps a window and all fit: nothing scales with the budget
            pages = max(self.window_pages) if spent <= budget else 0
        return int(pages), [int(w) if f else int(pages) for w, f in zip(self.window_pages, fixed)]

    def _profile(self, step_tokens: int, sample_rows: int, graph_rows: int, fraction: float, group_bytes: list[int]) -> dict:
        """How many pages fit beside what a step needs, measured, not estimated (as the reference sizes
        its pool, miniserve/engine/model_runner.py:152-203): on a probe pool just large enough, run the
        largest step (``step_tokens`` tokens of one request) and the largest sampling call
        (``sample_rows`` rows with a nucleus), read the allocator's peak, then a decode step of
        ``graph_rows`` rows, whose buffers every captured graph keeps for itself. The pool gets
        ``fraction`` of what is free beyond those."""
        ops = self.model.rt.ops
        rows = max(sample_rows, graph_rows, 1)
        probe_pages = max(-(-step_tokens // self.page_size) + 1, rows)
        per_group = [probe_pages for _ in self.layout.groups]
        cache = CacheManager(self.layout, self.page_size, per_group, rows, step_tokens, **self._allocator_kw())
        pool = KVPool(self.layout, self.page_size, per_group, rows, self.model.dtype, self.device)
        builder = BatchBuilder(self.device, len(self.layout.groups))

        def peak_of(fn) -> int:
            torch.cuda.synchronize(self.device)
            base = torch.cuda.memory_allocated(self.device)
            torch.cuda.reset_peak_memory_stats(self.device)
            fn()
            torch.cuda.synchronize(self.device)
            return torch.cuda.max_memory_allocated(self.device) - base

        def run(step_rows):
            starts = [r.cache.num_tokens for r in step_rows]
            for r in step_rows:
                cache.extend(r.cache, len(r.tokens))
            self.model.forward(builder.build(step_rows, starts), pool)

        def biggest_step():
            rc = cache.acquire()
            run([StepRow(rc, [0] * step_tokens, [step_tokens - 1])])
            cache.release(rc)
            logits = torch.zeros((sample_rows, self.model.vocab_size), dtype=torch.float32, device=self.device)
            ones = torch.ones((sample_rows,), dtype=torch.float32, device=self.device)
            ints = torch.arange(sample_rows, dtype=torch.int32, device=self.device)
            ops.sample_rows(logits, ones, ones * 0.9, ints, ints)

        def decode_step():
            handles = [cache.acquire() for _ in range(graph_rows)]
            run([StepRow(rc, [0], [0]) for rc in handles])
            for rc in handles:
                cache.release(rc)

        peak = peak_of(biggest_step)
        graph_step = peak_of(decode_step) if graph_rows else 0
        del pool, cache, builder
        torch.cuda.empty_cache()
        free, total = torch.cuda.mem_get_info(self.device)
        # Graphs of different table widths are captured as they are needed and each keeps its step's buffers.
        graph_reserve = 4 * graph_step
        max_pages, per_group = self.split_bytes(int(fraction * (free - peak - graph_reserve)), group_bytes)
        if max_pages < 1:
            raise RuntimeError(f"no memory left for the cache pool: {free} bytes free, a step peaks at {peak}")
        return {"profile_tokens": step_tokens, "profile_sample_rows": sample_rows, "peak_activation_bytes": peak,
                "decode_step_bytes": graph_step, "graph_reserve_bytes": graph_reserve, "free_bytes": free,
                "total_bytes": total, "max_pages": max_pages, "pages_per_group": per_group}

    # ------------------------------------------------------------------ request handles

    def acquire(self) -> RequestCache:
        return self.cache.acquire()

    def release(self, rc: RequestCache) -> None:
        self.cache.release(rc)

    # ------------------------------------------------------------------ the step function

    def step(self, rows: list[StepRow], feed_from: torch.Tensor | None = None) -> torch.Tensor | None:
        """Run one batch. Each row's tokens continue its cache at position ``cache.num_tokens``.
        Returns float32 logits ``[sum(len(row.want)), vocab]`` in row order (None if nothing is
        wanted). Raises ``OutOfBlocks`` with every table unchanged if the pool cannot hold the step.
        ``feed_from``: int32 device tensor of tokens an earlier step sampled; a row with ``feed = i``
        runs ``feed_from[i]`` as its last token (the host need not have read it back)."""
        if not rows:
            return None
        total = sum(len(r.tokens) for r in rows)
        if total > MAX_STEP_TOKENS:
            raise ValueError(f"a step of {total} tokens: one step carries at most {MAX_STEP_TOKENS}; cut the prompt into portions")
        vocab = self.model.vocab_size
        seen = set()
        for r in rows:
            if id(r.cache) in seen:
                raise ValueError("a request appears twice in one step")
            seen.add(id(r.cache))
            if not r.tokens:
                raise ValueError("a row without tokens")
            known = r.tokens if r.feed is None else r.tokens[:-1]
            if known and (min(known) < 0 or max(known) >= vocab):
                raise ValueError(f"token id out of range [0, {vocab})")
            if r.feed is not None:
                if feed_from is None or not 0 <= r.feed < feed_from.shape[0]:
                    raise ValueError("a row is fed from the device but no such token was given")
                r.tokens = known + [0]
            if r.want and not (0 <= min(r.want) and max(r.want) < len(r.tokens)):
                raise ValueError("wanted place outside the row's tokens")
        need = [0] * self.cache.num_groups
        for r in rows:
            for g, k in enumerate(self.cache.pages_needed(r.cache, len(r.tokens))):
                need[g] += k
        for g, (k, free) in enumerate(zip(need, self.cache.free_pages())):
            if k > free:
                raise OutOfBlocks(f"group {g}: the step needs {k} free pages, {free} free")
        starts = [r.cache.num_tokens for r in rows]
        for r in rows:
            self.cache.extend(r.cache, len(r.tokens))
        if self.graphs is not None and self.graphs.usable(rows):
            logits = self.graphs.run(rows, starts, feed_from)
            self.graph_steps += 1
            self._last = self.graphs.latest
        else:
            batch = self.builder.build(rows, starts)
            if batch.feed is not None:
                self.model.rt.ops.feed_tokens(batch.token_ids, batch.row_start, batch.feed, feed_from)
            logits = self.model.forward(batch, self.pool)
            self._last = batch
        for r in rows:
            self.cache.advance(r.cache)
        self.steps += 1
        return logits

    def repeat_last_step(self) -> None:
        """Run the latest step's model pass once more on the inputs it had: the same kernels over the same
        tokens at the same places (they write what is there already), nothing advances and nothing is
        returned. Keeps the device at the step's load without spending context: a warm-up at a fixed
        sequence length. Only before the next ``step``."""
        if self._last is None:
            raise RuntimeError("no step has run yet")
        graph = getattr(self._last, "graph", None)
        if graph is not None:
            graph.replay()
        else:
            self.model.forward(self._last, self.pool)
