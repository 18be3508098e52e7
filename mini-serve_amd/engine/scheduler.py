"""Batch assembly: which requests run in the next step, and what happens when pages run out.

Two modes, as in the reference (miniserve/engine/scheduler.py:1-49):

* ``chunked_prefill_size == 0``: prefill first. Waiting requests are admitted in order until the
  prefill token budget is spent (the first one even if it alone exceeds it); otherwise every
  running request decodes one token. A batch is all prefill or all decode.
* ``chunked_prefill_size > 0``: decode first. Every decoding request gets its token; the rest of the
  step's token budget goes to portions of prompts, first of requests part-way through their
  prefill, then of newly admitted ones. No step runs more tokens than the budget.

Pages. Admission takes nothing physically; it budgets: a request is admitted only if what it may
still draw until its prefill plus one decode token is in (per cache group, net of what windowed
groups give back) fits beside what the running requests may still draw. Admission stops at the
first request that does not fit: no skipping ahead. When the running requests' next step does not
fit, requests are preempted newest first (never the oldest): pages and state slot go back, the
request keeps its output and returns to the front of the waiting queue to be prefilled again
(prompt + output). No deadlock: a request that cannot fit the pool alone is refused at submission,
and the oldest running request always proceeds.
"""

from __future__ import annotations

import enum
from collections import deque
from dataclasses import dataclass, field

from .policy import FCFS
from .request import Request, RequestState


class Phase(enum.Enum):
    PREFILL = "prefill"
    DECODE = "decode"
    MIXED = "mixed"


@dataclass
class Batch:
    phase: Phase
    requests: list
    starts: list  # tokens whose cache exists before this step, per request
    extend_lens: list  # new tokens this step, per request
    num_decode: int  # rows [0, num_decode) are decode rows
    preempted: list = field(default_factory=list)

    def completes(self) -> list:
        """Rows that reach the end of their sequence this step and so sample a token."""
        return [s + n == r.seq_len for r, s, n in zip(self.requests, self.starts, self.extend_lens)]

    @property
    def num_tokens(self) -> int:
        return sum(self.extend_lens)


def _add(a, b):
    return [x + y for x, y in zip(a, b)]


class Scheduler:
    def __init__(self, max_running=64, max_prefill_tokens=8192, cache=None, chunked_prefill_size=0, policy=None):
        if max_running < 1 or max_prefill_tokens < 1:
            raise ValueError("max_running and max_prefill_tokens must be positive")
        if chunked_prefill_size < 0:
            raise ValueError(f"chunked_prefill_size must be >= 0, got {chunked_prefill_size}")
        if cache is None:
            raise ValueError("the scheduler budgets against a cache manager")
        self.max_running = max_running
        self.max_prefill_tokens = max_prefill_tokens
        self.cache = cache
        self.chunked_prefill_size = chunked_prefill_size
        self.policy = policy if policy is not None else FCFS()
        self.waiting: deque = deque()
        self.running: list = []  # admission order
        self.num_preemptions = 0
        self.stats = dict(first_tokens=0, re_tokens=0)

    # ------------------------------------------------------------------ submission

    def add(self, req: Request) -> None:
        if req.state is not RequestState.WAITING:
            raise ValueError(f"request {req.rid} is {req.state.name}, expected WAITING")
        if not self.cache.fits_alone(req.max_len):
            held = [t * self.cache.page_size for t in self.cache.total_pages()]
            raise ValueError(f"request {req.rid} needs up to {req.max_len} tokens of cache, the pool holds {held}")
        self.waiting.append(req)

    @property
    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def retire(self, req: Request) -> None:
        if not req.is_done:
            raise ValueError(f"request {req.rid} is {req.state.name}, not done")
        if req in self.running:
            self.running.remove(req)
        elif req in self.waiting:
            self.waiting.remove(req)

    # ------------------------------------------------------------------ budgets

    def _zero(self):
        return [0] * self.cache.num_groups

    @staticmethod
    def _decodes(r: Request) -> bool:
        return r.state is RequestState.DECODE and not r.reached_max_tokens

    def _outstanding(self, reqs) -> list:
        """Pages per group ``reqs`` may still draw before any of them finishes: the next token of
        each decoding request, the rest of the prefill plus one token of each prefilling one."""
        need = self._zero()
        for r in reqs:
            if self._decodes(r):
                need = _add(need, self.cache.pages_needed(r.cache, 1))
            elif r.state is RequestState.PREFILL:
                need = _add(need, self.cache.outstanding(r.cache, r.seq_len + 1))
        return need

    def _exceeds(self, need) -> bool:
        return any(n > f for n, f in zip(need, self.cache.free_pages()))

    def _try_admit(self, req: Request, reserved) -> list | None:
        """Acquire a cache handle for ``req`` if its whole prefill plus one token fits beside the
        running requests and ``reserved``; returns its need, or None (nothing is left behind)."""
        rc = self.cache.acquire()
        need = self.cache.outstanding(rc, req.seq_len + 1)
        spoken = _add(self._outstanding(self.running), reserved)
        if any(n > f - s for n, f, s in zip(need, self.cache.free_pages(), spoken)):
            self.cache.release(rc)
            return None
        req.cache = rc
        return need

    def _admitted(self, req: Request) -> None:
        self.waiting.remove(req)
        req.transition(RequestState.PREFILL)
        self.stats["first_tokens" if req.num_preemptions == 0 else "re_tokens"] += req.seq_len

    # ------------------------------------------------------------------ preemption

    def _pick_victim(self, pool) -> Request:
        candidates = [r for r in pool if r is not self.running[0]]
        assert candidates, "a lone request does not fit in the pool"
        return self.policy.pick_victim(candidates)

    def _preempt(self, req: Request) -> None:
        req.transition(RequestState.WAITING)
        self.cache.release(req.cache)
        req.cache = None
        self.running.remove(req)
        self.waiting.appendleft(req)
        req.num_preemptions += 1
        self.num_preemptions += 1

    # ------------------------------------------------------------------ scheduling

    def schedule(self) -> Batch | None:
        if self.chunked_prefill_size:
            return self._schedule_chunked()
        admitted = self._admit_whole()
        if admitted:
            self.running.extend(admitted)
            return Batch(Phase.PREFILL, admitted, [0] * len(admitted), [r.seq_len for r in admitted], 0)
        decoding = [r for r in self.running if self._decodes(r)]
        preempted = []
        while self._exceeds(self._outstanding(decoding)):
            victim = self._pick_victim(decoding)
            decoding.remove(victim)
            self._preempt(victim)
            preempted.append(victim)
        if not decoding:
            return None
        return Batch(Phase.DECODE, decoding, [r.seq_len - 1 for r in decoding], [1] * len(decoding), len(decoding), preempted)

    def _admit_whole(self) -> list:
        admitted = []
        budget = self.max_prefill_tokens
        reserved = self._zero()
        for req in self.policy.order(self.waiting):
            if len(self.running) + len(admitted) >= self.max_running:
                break
            if admitted and req.seq_len > budget:
                break  # the first request is admitted even if it alone exceeds the budget
            need = self._try_admit(req, reserved)
            if need is None:
                break
            reserved = _add(reserved, need)
            self._admitted(req)
            admitted.append(req)
            budget -= req.seq_len
        return admitted

    def _schedule_chunked(self) -> Batch | None:
        preempted = []
        while self._exceeds(self._outstanding(self.running)):
            assert len(self.running) > 1, "a lone request does not fit in the pool"
            victim = self._pick_victim(self.running)
            self._preempt(victim)
            preempted.append(victim)
        budget = self.chunked_prefill_size
        rows = [(r, r.seq_len - 1, 1) for r in self.running if self._decodes(r)]
        num_decode = len(rows)
        budget -= num_decode
        for r in self.running:
            if r.state is RequestState.PREFILL and budget > 0:
                start = r.cache.num_tokens
                n = min(r.seq_len - start, budget)
                rows.append((r, start, n))
                budget -= n
        for req in self.policy.order(self.waiting) if budget > 0 else ():
            if budget <= 0 or len(self.running) >= self.max_running:
                break
            if self._try_admit(req, self._zero()) is None:
                break
            self._admitted(req)
            self.running.append(req)
            n = min(req.seq_len, budget)
            rows.append((req, 0, n))
            budget -= n
        if not rows:
            return None
        phase = Phase.DECODE if num_decode == len(rows) else Phase.PREFILL if num_decode == 0 else Phase.MIXED
        return Batch(phase, [r for r, _, _ in rows], [s for _, s, _ in rows], [n for _, _, n in rows], num_decode, preempted)
