"""The engine loop: ``step()`` = schedule -> one step of the model -> sample -> read back -> retire.

Interface in the reference's manner (miniserve/engine/engine.py:41-211): ``Engine(model, **options)``,
``add_request(prompt_ids, SamplingParams) -> Request``, ``step() -> Batch | None``, ``abort(rid)``,
``generate(prompts, params) -> list[list[int]]``, ``has_unfinished``, ``logits_hook``. Token ids in,
token ids out; the engine never tokenizes.

Each step is synchronous: the sampled tokens are read back (one copy of ``[rows]`` int32) before the
next step is scheduled. Only the rows that complete their sequence in a step ask for logits and are
sampled; a portion of a prompt that stops short asks for none (the reference computes and discards
a row for it, miniserve/engine/engine.py:156-172).
"""

from __future__ import annotations

import itertools
import random
from collections.abc import Sequence

from .batch import StepRow
from .policy import make_policy
from .request import Request, RequestState, SamplingParams
from .scheduler import Batch, Scheduler

DEFAULT_CHUNKED_PREFILL = 2048


class Engine:
    def __init__(
        self,
        model,
        max_running: int = 64,
        max_prefill_tokens: int = 8192,
        kv_pool_tokens: int | None = None,
        seed: int = 0,
        runner=None,
        chunked_prefill_size: int | None = None,
        schedule_policy: str = "fcfs",
        page_size: int = 16,
        kv_mem_fraction: float = 0.9,
        decode_graph: bool = True,
        decode_graph_max_bs: int | None = None,
        block_backend: str | None = None,
        sampler=None,
    ):
        """``kv_pool_tokens``: exact cache pool size in tokens (default: as large as memory allows).
        ``chunked_prefill_size``: token budget per step with prompts cut into portions and batched
        with decodes; 0 keeps whole prefills in prefill-only steps; default 2048.
        ``decode_graph``: replay captured HIP graphs for pure decode steps of up to
        ``decode_graph_max_bs`` requests (default ``max_running``).
        ``block_backend``: ``python`` or ``cpp`` page bookkeeping.
        ``seed``: seeds the sampling of requests submitted without a seed of their own, in
        submission order. ``runner``: use this model runner instead of building one for ``model``."""
        if chunked_prefill_size is None:
            chunked_prefill_size = DEFAULT_CHUNKED_PREFILL
        if runner is None:
            from ..cache.backend import allocator_class
            from .runner import ModelRunner

            runner = ModelRunner(
                model,
                page_size=page_size,
                kv_pool_tokens=kv_pool_tokens,
                kv_mem_fraction=kv_mem_fraction,
                max_running=max_running,
                max_step_tokens=chunked_prefill_size or max_prefill_tokens,
                allocator_class=allocator_class(block_backend),
                decode_graph=decode_graph,
                decode_graph_max_bs=decode_graph_max_bs,
            )
        self.runner = runner
        self.scheduler = Scheduler(
            max_running, max_prefill_tokens, cache=runner.cache, chunked_prefill_size=chunked_prefill_size,
            policy=make_policy(schedule_policy),
        )
        if sampler is None:
            from ..sampling.sampler import Sampler

            sampler = Sampler(runner.device, runner.model.vocab_size)
        self.sampler = sampler
        self.requests: dict = {}  # unfinished requests by id
        self._rids = itertools.count()
        self._seeds = random.Random(seed)
        self.logits_hook = None  # called with (batch, logits of the completing rows) before sampling
        self.launched: Batch | None = None
        self.num_steps = 0

    # ------------------------------------------------------------------ requests

    def add_request(self, prompt_ids: Sequence[int], params: SamplingParams) -> Request:
        req = Request(next(self._rids), list(prompt_ids), params)
        req.seed = params.seed if params.seed is not None else self._seeds.randrange(2**32)
        self.scheduler.add(req)
        self.requests[req.rid] = req
        return req

    def abort(self, rid: int) -> None:
        req = self.requests.get(rid)
        if req is None:
            return  # already finished or never existed
        req.transition(RequestState.ABORTED)
        self._retire(req)

    @property
    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished

    # ------------------------------------------------------------------ the loop

    def step(self) -> Batch | None:
        """Run one step; returns the batch it ran (its requests now carry their new tokens), or None
        when idle."""
        batch = self.scheduler.schedule()
        self.launched = batch
        if batch is None:
            return None
        completes = batch.completes()
        rows = [
            StepRow(r.cache, r.token_slice(s, n), [n - 1] if done else [])
            for r, s, n, done in zip(batch.requests, batch.starts, batch.extend_lens, completes)
        ]
        logits = self.runner.step(rows)
        self.num_steps += 1
        sampling = [r for r, done in zip(batch.requests, completes) if done]
        if not sampling:
            return batch
        if self.logits_hook is not None:
            self.logits_hook(batch, logits)
        tokens = self.sampler.sample(logits, self.sampler.prepare(sampling)).tolist()
        for r, tok in zip(sampling, tokens):
            r.output_ids.append(tok)
            if r.state is RequestState.PREFILL:
                r.transition(RequestState.DECODE)
            if r.should_stop():
                r.transition(RequestState.FINISHED)
                self._retire(r)
        return batch

    def _retire(self, req: Request) -> None:
        if req.cache is not None:
            self.runner.release(req.cache)
            req.cache = None
        self.scheduler.retire(req)
        del self.requests[req.rid]

    def generate(self, prompts: Sequence[Sequence[int]], params: SamplingParams) -> list:
        """Offline helper: submit all prompts at once and run to completion."""
        reqs = [self.add_request(p, params) for p in prompts]
        while self.has_unfinished:
            self.step()
        return [r.output_ids for r in reqs]
