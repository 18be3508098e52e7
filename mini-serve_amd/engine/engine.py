"""The engine loop: ``step()`` = schedule -> one step of the model -> sample -> read back -> retire,
with the read-back lagging one step behind by default.

Interface in the reference's manner (miniserve/engine/engine.py:41-211): ``Engine(model, **options)``,
``add_request(prompt_ids, SamplingParams) -> Request``, ``step() -> Batch | None``, ``abort(rid)``,
``generate(prompts, params) -> list[list[int]]``, ``has_unfinished``, ``logits_hook``. Token ids in,
token ids out; the engine never tokenizes.

Overlap (one-step lag, miniserve/engine/engine.py:9-21,137-147,167-198): step t + 1 is scheduled and
launched before the tokens of step t are read back, so the device never waits for the host's
bookkeeping. Until then a sampled token is only counted by its request (``Request.in_flight``); the next
step takes it from the device tensor the sampler left (``Request.feed``, ``StepRow.feed``). What the host learns one
step late is a stop token: the request has then run one step too many, and the token that step
sampled for it is dropped. Stops by length are known in advance and cost nothing. With
``overlap=False`` every step's tokens are read back (one copy of ``[rows]`` int32) before the next
step is scheduled. Only the rows that complete their sequence in a step ask for logits and are
sampled; a portion of a prompt that stops short asks for none (the reference computes and discards
a row for it, miniserve/engine/engine.py:156-172).
"""

from __future__ import annotations

import itertools
import random
from collections.abc import Sequence
from dataclasses import dataclass

import torch

from .batch import StepRow
from .policy import make_policy
from .request import Request, RequestState, SamplingParams
from .scheduler import Batch, Scheduler


@dataclass
class _Launched:
    """A step that has been handed to the device (miniserve/engine/engine.py:214-221)."""

    batch: Batch
    sampling: list  # the requests that sample a token in this step, in row order
    tokens: object = None  # int32 [len(sampling)] where the sampler left them
    host: object = None  # the same on the host once ``ready`` has passed
    ready: object = None  # event after the copy to the host (None: ``host`` is valid already)

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
        overlap: bool = True,
    ):
        """``kv_pool_tokens``: exact cache pool size in tokens (default: as large as memory allows).
        ``chunked_prefill_size``: token budget per step with prompts cut into portions and batched
        with decodes; 0 keeps whole prefills in prefill-only steps; default 2048.
        ``decode_graph``: replay captured HIP graphs for pure decode steps of up to
        ``decode_graph_max_bs`` requests (default ``max_running``).
        ``block_backend``: ``python`` or ``cpp`` page bookkeeping.
        ``seed``: seeds the sampling of requests submitted without a seed of their own, in
        submission order. ``runner``: use this model runner instead of building one for ``model``.
        ``overlap``: launch the next step before the tokens of this one are read back."""
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
                request_step_tokens=chunked_prefill_size or None,  # whole prompts run in one step, however long
                allocator_class=allocator_class(block_backend),
                decode_graph=decode_graph,
                decode_graph_max_bs=decode_graph_max_bs,
            )
        self.runner = runner
        spec = getattr(getattr(runner, "model", None), "spec", None)
        self.scheduler = Scheduler(
            max_running, max_prefill_tokens, cache=runner.cache, chunked_prefill_size=chunked_prefill_size,
            policy=make_policy(schedule_policy), max_step_tokens=getattr(runner, "max_step_tokens_limit", None),
            max_position=getattr(spec, "max_position", None),
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
        self.overlap = overlap
        self._inflight: _Launched | None = None  # launched, tokens not read back yet
        self.dropped_tokens = 0  # sampled for a request that had already ended (overlap only)

    # ------------------------------------------------------------------ requests

    def add_request(self, prompt_ids: Sequence[int], params: SamplingParams) -> Request:
        seed = params.seed if params.seed is not None else self._seeds.randrange(2**32)
        req = Request(next(self._rids), prompt_ids, params, seed)
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
        """Schedule and launch one step; read back, and return the batch of, the step whose tokens
        are due: this one without overlap, the previous one with it (None when there is none)."""
        prev, self._inflight = self._inflight, None
        batch = self.scheduler.schedule()
        self.launched = batch
        launched = self._launch(batch, prev) if batch is not None else None
        if not self.overlap:
            if prev is not None:  # ``overlap`` was switched off between two steps: the step before is still due
                self._finish(prev)
            return self._finish(launched) if launched is not None else None
        self._inflight = launched
        return self._finish(prev) if prev is not None else None

    def _launch(self, batch: Batch, prev: _Launched | None) -> _Launched:
        completes = batch.completes()
        rows, fed = [], False
        for (r, start, n), done in zip(batch.rows, completes):
            tokens, feed = r.step_tokens(start, n)  # feed: the row's last token is still in ``prev.tokens``
            fed = fed or feed is not None
            rows.append(StepRow(r.cache, tokens, [n - 1] if done else [], feed))
        logits = self.runner.step(rows, feed_from=prev.tokens) if fed else self.runner.step(rows)
        self.num_steps += 1
        sampling = [r for (r, _, _), done in zip(batch.rows, completes) if done]
        launched = _Launched(batch, sampling)
        if not sampling:
            return launched
        if self.logits_hook is not None:
            self.logits_hook(batch, logits)
        launched.tokens = self.sampler.sample(logits, self.sampler.prepare(sampling))
        if launched.tokens.is_cuda:
            launched.host = torch.empty(launched.tokens.shape, dtype=launched.tokens.dtype, pin_memory=True)
            launched.host.copy_(launched.tokens, non_blocking=True)
            launched.ready = torch.cuda.Event()
            launched.ready.record()
        else:
            launched.host = launched.tokens
        for i, r in enumerate(sampling):
            r.sampled(i)
            if r.state is RequestState.PREFILL:
                r.transition(RequestState.DECODE)
            if r.sampled_all:
                # Its last step is under way: the pages go back now, not at the read-back. Whoever gets them
                # next writes them in a later step, behind this one in the stream.
                self.runner.release(r.cache)
                r.cache = None
        return launched

    def _finish(self, launched: _Launched) -> Batch:
        """Read the step's tokens back, append them to their requests, end what they end."""
        if not launched.sampling:
            return launched.batch
        if launched.ready is not None:
            launched.ready.synchronize()
        for r, tok in zip(launched.sampling, launched.host.tolist()):
            if r.is_done:  # aborted, or ended by the token before this one: this one ran past the end
                self.dropped_tokens += 1
                continue
            if r.read_back(tok):
                r.forget_in_flight()  # counted as dropped when the step that sampled it is read back
                r.transition(RequestState.FINISHED)
                self._retire(r)
        return launched.batch

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
