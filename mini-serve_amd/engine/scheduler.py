"""Which requests run in the next step, with how many tokens each, and who gives way when pages run out.

One pass builds every step, whatever the mode. The step has a token budget and the cache has, per
layer group, a vector of free pages; both are spent in a fixed order:

1. **Make room.** If the running requests' own next step does not fit the free pages, the newest
   running request that holds pages gives way (never the oldest): its pages and state slot go back,
   it keeps its tokens and returns to the front of the queue, to be prefilled again over prompt +
   output. Repeated until the rest fits.
2. **Decode rows**: one token for every request that is decoding.
3. **Portions** of prompts that are part-way in (only with ``chunked_prefill_size > 0``).
4. **Admissions**, in the policy's order, while the token budget lasts. A request is admitted only
   if the pages it may still draw until its whole prefill and one more token are in (per group, net of
   what windowed groups give back) fit beside what every running request may still draw. Nothing
   is taken physically: pages are drawn step by step by the step function. The first request that
   does not fit ends the pass: no skipping ahead.

``chunked_prefill_size > 0`` (the default): the budget is that many tokens, decode rows are served
first and count against it, prompts are cut to what is left, and one step mixes all three kinds
of rows. ``chunked_prefill_size == 0``: prompts run whole, the budget (``max_prefill_tokens``) only
limits how many share a step (the first is admitted even if it alone exceeds it), and a step that
admits anything runs only the admitted prompts; decoding requests wait for the next one. These are the
reference's two schedules (miniserve/engine/scheduler.py:1-49,156-279) and its rows step for step
(tests/test_engine.py:141-202,286-345,355-439).

No deadlock: a request that could not fit the pool alone is refused at submission, and the oldest
request that holds pages always proceeds. A request whose every token has been sampled holds no
pages any more (the engine gives them back at the launch of its last step, not at the read-back),
so it never stands in anybody's way; the reference frees such requests first when pages run out
(:281-292).
"""

from __future__ import annotations

import enum
from collections import deque
from dataclasses import dataclass, field

import numpy as np

from .policy import FCFS
from .request import Request, RequestState


class Phase(enum.Enum):
    PREFILL = "prefill"
    DECODE = "decode"
    MIXED = "mixed"


@dataclass
class Batch:
    """One step's rows: ``(request, tokens already in its cache, new tokens)``, decode rows first."""

    rows: list
    num_decode: int
    preempted: list = field(default_factory=list)

    @property
    def phase(self) -> Phase:
        if self.num_decode == len(self.rows):
            return Phase.DECODE
        return Phase.MIXED if self.num_decode else Phase.PREFILL

    @property
    def requests(self) -> list:
        return [r for r, _, _ in self.rows]

    @property
    def starts(self) -> list:
        return [s for _, s, _ in self.rows]

    @property
    def extend_lens(self) -> list:
        return [n for _, _, n in self.rows]

    @property
    def num_tokens(self) -> int:
        return sum(n for _, _, n in self.rows)

    def completes(self) -> list:
        """Per row: whether it reaches the end of its sequence in this step, and so samples a token."""
        return [s + n == r.seq_len for r, s, n in self.rows]


class Scheduler:
    def __init__(self, max_running=64, max_prefill_tokens=8192, cache=None, chunked_prefill_size=0, policy=None,
                 max_step_tokens=None, max_position=None):
        """``max_step_tokens``: most tokens the step function takes at once (None: no limit);
        ``max_position``: longest sequence the model is meant for (None: no limit)."""
        if max_running < 1 or max_prefill_tokens < 1:
            raise ValueError("max_running and max_prefill_tokens must be positive")
        if max_step_tokens is not None and max(chunked_prefill_size, 0 if chunked_prefill_size else max_prefill_tokens) > max_step_tokens:
            raise ValueError(f"a step carries at most {max_step_tokens} tokens: chunked_prefill_size / max_prefill_tokens exceed it")
        self.max_step_tokens = max_step_tokens
        self.max_position = max_position
        if chunked_prefill_size < 0:
            raise ValueError(f"chunked_prefill_size must be >= 0, got {chunked_prefill_size}")
        if cache is None:
            raise ValueError("the scheduler budgets against a cache manager")
        self.max_running = max_running
        self.max_prefill_tokens = max_prefill_tokens
        self.chunk = chunked_prefill_size
        self.cache = cache
        self.policy = policy if policy is not None else FCFS()
        self.waiting: deque = deque()
        self.running: list = []  # in admission order
        self.num_preemptions = 0
        self.stats = {"first_tokens": 0, "re_tokens": 0}  # prefill tokens of first admissions / of admissions after a preemption

    @property
    def chunked_prefill_size(self) -> int:
        return self.chunk

    # ------------------------------------------------------------------ in and out

    def add(self, req: Request) -> None:
        if req.state is not RequestState.WAITING:
            raise ValueError(f"request {req.rid} is {req.state.name}; only a waiting request can be submitted")
        if self.max_position is not None and req.max_len > self.max_position:
            # the reference's server refuses the same (miniserve/server/__main__.py:29-33)
            raise ValueError(f"request {req.rid}: prompt + max_new_tokens = {req.max_len} tokens exceed the model's "
                             f"max_position_embeddings = {self.max_position}")
        if not self.chunk and self.max_step_tokens is not None and req.max_len - 1 > self.max_step_tokens:
            raise ValueError(f"request {req.rid}: a sequence of up to {req.max_len - 1} tokens cannot run whole, one step carries "
                             f"at most {self.max_step_tokens}: use chunked prefill")
        # Prefilled again after a preemption it runs up to max_len - 1 tokens; whole prompts run in one step.
        if not self.cache.fits_alone(req.max_len, self.chunk or req.max_len):
            held = [t * self.cache.page_size for t in self.cache.total_pages()]
            raise ValueError(f"request {req.rid} needs up to {req.max_len} tokens of cache, the pool holds {held}")
        self.waiting.append(req)

    def retire(self, req: Request) -> None:
        """Forget a request that has finished or was aborted, wherever it stands."""
        if not req.is_done:
            raise ValueError(f"request {req.rid} is {req.state.name}: only finished or aborted requests leave")
        for queue in (self.running, self.waiting):
            if req in queue:
                queue.remove(req)
                return

    @property
    def has_unfinished(self) -> bool:
        return bool(self.running) or bool(self.waiting)

    # ------------------------------------------------------------------ page vectors

    def _step_of(self, req: Request) -> int:
        """Most tokens a step carries for ``req``: what bounds the pages a windowed group holds for it."""
        return self.chunk or req.seq_len

    def _may_draw(self, reqs) -> np.ndarray:
        """Pages per group that ``reqs`` may still take before any of them ends: the next token of each
        decoding request, the rest of the prefill and one token of each prefilling one."""
        need = np.zeros(self.cache.num_groups, dtype=np.int64)
        for r in reqs:
            if r.cache is None:
                continue  # everything sampled: it holds nothing and runs no more
            if r.state is RequestState.PREFILL:
                need += self.cache.outstanding(r.cache, r.seq_len + 1, self._step_of(r))
            elif r.decodes:
                need += self.cache.pages_needed(r.cache, 1)
        return need

    def _free(self) -> np.ndarray:
        return np.asarray(self.cache.free_pages(), dtype=np.int64)

    # ------------------------------------------------------------------ the pass

    def schedule(self) -> Batch | None:
        preempted = self._make_room()
        budget = self.chunk or self.max_prefill_tokens
        decode_rows = [(r, r.seq_len - 1, 1) for r in self.running if r.decodes]
        rows = []
        if self.chunk:
            rows = list(decode_rows)
            budget -= len(rows)
            for r in self.running:
                if budget <= 0:
                    break
                if r.state is RequestState.PREFILL:
                    done = r.cache.num_tokens
                    n = min(r.seq_len - done, budget)
                    rows.append((r, done, n))
                    budget -= n
        admitted = self._admit(budget)
        num_decode = len(decode_rows)
        if self.chunk:
            rows += admitted
        elif admitted:
            rows, num_decode = admitted, 0  # a step of whole prompts; decoding requests wait for the next one
        else:
            rows = decode_rows
        return Batch(rows, num_decode, preempted) if rows else None

    def _make_room(self) -> list:
        preempted = []
        while (self._may_draw(self.running) > self._free()).any():
            holding = [r for r in self.running if r.cache is not None]
            if len(holding) < 2:
                raise RuntimeError(
                    f"request {holding[0].rid if holding else None} does not fit the pool alone although it was admitted"
                )
            victim = self.policy.pick_victim(holding[1:])
            victim.transition(RequestState.WAITING)
            self.cache.release(victim.cache)
            victim.cache = None
            victim.num_preemptions += 1
            self.num_preemptions += 1
            self.running.remove(victim)
            self.waiting.appendleft(victim)
            preempted.append(victim)
        return preempted

    def _admit(self, budget: int) -> list:
        """Admit waiting requests in the policy's order; returns their rows ``(request, 0, tokens)``."""
        rows = []
        for req in self.policy.order(self.waiting):
            if len(self.running) >= self.max_running:
                break
            if self.chunk:
                if budget <= 0:
                    break
                n = min(req.seq_len, budget)
            else:
                n = req.seq_len
                if rows and n > budget:
                    break  # only the first prompt of a step may exceed the budget
            handle = self.cache.acquire()
            need = self.cache.outstanding(handle, req.seq_len + 1, self._step_of(req))
            if (need > self._free() - self._may_draw(self.running)).any():
                self.cache.release(handle)  # nothing stays behind a refused admission
                break
            req.cache = handle
            req.transition(RequestState.PREFILL)
            self.waiting.remove(req)
            self.running.append(req)
            self.stats["re_tokens" if req.num_preemptions else "first_tokens"] += req.seq_len
            rows.append((req, 0, n))
            budget -= n
        return rows
