"""A CPU stand-in for the model runner, for tests of the scheduler and the engine loop: the real
cache manager and tables underneath, but "keys and values" that are just (token, position) pairs
per slot. Every step writes the new tokens through the tables, then reads each wanted sequence
back through its table, checks that it finds positions 0..n-1 of exactly the request's tokens
(so a wrong table, a reused page that was not rewritten, or a wrong position shows), and returns
pseudo-logits that are a pure function of the sequence so far. The reference tests its engine the
same way (tests/test_engine.py:481-559)."""

from __future__ import annotations

import zlib

import numpy as np
import torch

from miniserve_amd.cache import CacheLayout, CacheManager, OutOfBlocks
from miniserve_amd.cache.backend import allocator_class
from miniserve_amd.parts.base import KVNeed
from miniserve_amd.parts.model import CacheSlotNeed


class _ToyModel:
    def __init__(self, vocab):
        self.vocab_size = vocab


def pseudo_logits(tokens, vocab) -> np.ndarray:
    seed = zlib.crc32(np.asarray(tokens, dtype=np.int64).tobytes())
    return np.random.default_rng(seed).standard_normal(vocab).astype(np.float32) * 3


class ToyRunner:
    def __init__(self, num_pages, page_size=4, vocab=50, windows=(0,), max_running=8, max_step_tokens=None, backend="python"):
        needs = [CacheSlotNeed(i, KVNeed.keys_values(1, 16, w), None) for i, w in enumerate(windows)]
        self.layout = CacheLayout.from_needs(needs)
        self.cache = CacheManager(self.layout, page_size, [num_pages] * len(self.layout.groups), max_running,
                                  max_step_tokens, allocator_class=allocator_class(backend))
        self.page_size = page_size
        self.model = _ToyModel(vocab)
        self.device = torch.device("cpu")
        self.store = [dict() for _ in self.layout.groups]  # per group: slot -> (token, position)
        self.history = {}  # id(cache) -> tokens fed so far
        self.steps = 0
        self.max_tokens_in_a_step = 0

    def acquire(self):
        return self.cache.acquire()

    def release(self, rc):
        self.history.pop(id(rc), None)
        self.cache.release(rc)

    def step(self, rows, feed_from=None):
        for r in rows:  # a token that is "still on the device": the last of the row
            if getattr(r, "feed", None) is not None:
                r.tokens = list(r.tokens[:-1]) + [int(feed_from[r.feed])]
        assert all(t >= 0 for r in rows for t in r.tokens), "a placeholder reached the model"
        need = [0] * self.cache.num_groups
        for r in rows:
            for g, k in enumerate(self.cache.pages_needed(r.cache, len(r.tokens))):
                need[g] += k
        if any(k > f for k, f in zip(need, self.cache.free_pages())):
            raise OutOfBlocks("the step does not fit")
        self.max_tokens_in_a_step = max(self.max_tokens_in_a_step, sum(len(r.tokens) for r in rows))
        out = []
        for r in rows:
            rc = r.cache
            start = rc.num_tokens
            if start == 0:
                self.history[id(rc)] = []  # a fresh handle (ids of dead handles come back)
            hist = self.history[id(rc)]
            assert len(hist) == start, "a row must continue where its cache ends"
            self.cache.extend(rc, len(r.tokens))
            for g, table in enumerate(rc.tables):
                for i, (tok, slot) in enumerate(zip(r.tokens, table.tail_slots(len(r.tokens)))):
                    self.store[g][slot] = (tok, start + i)
            hist.extend(r.tokens)
            for k in r.want:
                upto = start + k + 1
                for g, (grp, table) in enumerate(zip(self.layout.groups, rc.tables)):
                    lo = max(0, upto - grp.window) if grp.window else 0
                    seen = [self.store[g][table.slot(p)] for p in range(lo, upto)]
                    assert seen == [(hist[p], p) for p in range(lo, upto)], "the cache does not hold the sequence"
                out.append(pseudo_logits(hist[:upto], self.model.vocab_size))
        for r in rows:
            self.cache.advance(r.cache)
        self.steps += 1
        return torch.from_numpy(np.stack(out)) if out else None


class ToySampler:
    """The plain sampler on CPU logits, with the engine's interface."""

    def __init__(self):
        from plain import qwen3_plain as P

        self.P = P

    def prepare(self, requests):
        return [(r.params.temperature, r.seed, r.seq_len, r.params.top_p) for r in requests]

    def sample(self, logits, args):
        rows = logits.numpy()
        return torch.tensor([self.P.sample(rows[i], *a) for i, a in enumerate(args)], dtype=torch.int32)


def run_alone(prompt, params, seed, vocab):
    """What a request produces by itself: the sampler over the pseudo-logits of its growing history."""
    from plain import qwen3_plain as P

    ids, out = list(prompt), []
    while len(out) < params.max_new_tokens:
        tok = P.sample(pseudo_logits(ids, vocab), params.temperature, seed, len(ids), params.top_p)
        out.append(tok)
        ids.append(tok)
        if tok in params.stop_token_ids:
            break
    return out
