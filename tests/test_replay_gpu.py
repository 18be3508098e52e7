"""Trace replay against the plain implementation: the same requests whole; most of each in one
step and the last 32 tokens one by one; in portions of changing size down to two tokens; and mixed,
up to four live requests, portions of some beside decoded tokens of others, in a pool so small
that pages are used again. In float32 and in bfloat16, on tiny models that differ in every size."""

from __future__ import annotations

import numpy as np
import pytest

from models import TINY, make_folder
from plain import qwen3_plain as P
from plain.model_folder import read_model_folder
from replay_util import Replay, round64
from tolerances import check_logits

pytestmark = pytest.mark.gpu

DTYPES = ("float32", "bfloat16")
LENGTHS = {
    "tinyA": [40, 7, 33, 64, 19, 90], "tinyB": [97, 3, 50, 65, 128, 31, 80], "tinyC": [100, 30, 77, 129, 48],
    "tinyD": [300, 1, 65, 130, 2, 47], "tinyE": [520, 33, 257, 64, 150],
}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_folder(root, name) for name in TINY}


@pytest.fixture(scope="module")
def truth(folders):
    """Per model: the requests' token ids and the plain implementation's logits at every position."""
    out = {}
    for name, folder in folders.items():
        cfg, w = read_model_folder(folder)
        rng = np.random.default_rng(sum(map(ord, name)))
        reqs = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in LENGTHS[name]]
        out[name] = (reqs, [P.logits(cfg, w, ids) for ids in reqs])
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(TINY))
def test_whole(name, dtype, folders, truth, tmp_path):
    reqs, want = truth[name]
    with Replay(folders[name], dtype, tmp_path / "out", max(round64(len(r)) for r in reqs)) as rp:
        for i, (ids, ref) in enumerate(zip(reqs, want)):
            got = rp.step([(f"r{i}", ids, range(len(ids)))], end=[f"r{i}"])
            check_logits(got, ref, dtype, f"{name} request {i} whole")
        assert rp.close() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(TINY))
def test_last_32_one_by_one(name, dtype, folders, truth, tmp_path):
    reqs, want = truth[name]
    with Replay(folders[name], dtype, tmp_path / "out", max(round64(len(r)) for r in reqs)) as rp:
        for i, (ids, ref) in enumerate(zip(reqs, want)):
            n = len(ids)
            head = max(n - 32, 1)
            got = rp.step([(f"r{i}", ids[:head], [head - 1])])
            check_logits(got, ref[head - 1 : head], dtype, f"{name} request {i} head")
            for p in range(head, n):
                got = rp.step([(f"r{i}", [ids[p]], [0])], end=[f"r{i}"] if p == n - 1 else [])
                check_logits(got, ref[p : p + 1], dtype, f"{name} request {i} position {p}")
            if head == n:
                rp.step([], end=[f"r{i}"])
        assert rp.close() == 0


PORTIONS = [5, 13, 32, 2, 7, 2, 21, 16, 3, 64]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(TINY))
def test_portions_of_changing_size(name, dtype, folders, truth, tmp_path):
    reqs, want = truth[name]
    with Replay(folders[name], dtype, tmp_path / "out", max(round64(len(r)) for r in reqs)) as rp:
        for i, (ids, ref) in enumerate(zip(reqs, want)):
            at, k = 0, i  # start the cycle elsewhere for every request
            while at < len(ids):
                n = min(PORTIONS[k % len(PORTIONS)], len(ids) - at)
                k += 1
                last = at + n == len(ids)
                got = rp.step([(f"r{i}", ids[at : at + n], range(n))], end=[f"r{i}"] if last else [])
                check_logits(got, ref[at : at + n], dtype, f"{name} request {i} portion at {at} of {n}")
                at += n
        assert rp.close() == 0


def mixed_schedule(lengths, seed):
    """Steps for up to four live requests: each live request gets a portion (prefill) or one token
    (the last 8 tokens of each request go one by one), some requests sit a step out, finished ones
    end and the next starts. Returns (steps, peak of live tokens rounded up per request)."""
    rng = np.random.default_rng(seed)
    fed = [0] * len(lengths)
    waiting = list(range(len(lengths)))
    live: list[int] = []
    steps = []
    peak = 0
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        peak = max(peak, sum(round64(lengths[i]) for i in live))
        entries, ends = [], []
        for i in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step
            left = lengths[i] - fed[i]
            n = 1 if left <= 8 else int(min(left - 8, rng.choice([2, 3, 5, 13, 17, 32, 40])))
            entries.append((i, fed[i], n))
            fed[i] += n
            if fed[i] == lengths[i]:
                ends.append(i)
                live.remove(i)
        if entries:
            steps.append((entries, ends))
    return steps, peak


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(TINY))
def test_mixed_with_page_reuse(name, dtype, folders, truth, tmp_path):
    reqs, want = truth[name]
    steps, peak = mixed_schedule([len(r) for r in reqs], seed=11)
    assert any(len(e) > 1 and min(n for _, _, n in e) == 1 and max(n for _, _, n in e) > 1 for e, _ in steps), \
        "the schedule must mix portions with single tokens"
    assert sum(round64(len(r)) for r in reqs) > peak, "the pool must be too small to hold all requests: pages are reused"
    with Replay(folders[name], dtype, tmp_path / "out", peak) as rp:
        for entries, ends in steps:
            got = rp.step([(f"r{i}", reqs[i][s : s + n], range(n)) for i, s, n in entries], end=[f"r{i}" for i in ends])
            at = 0
            for i, s, n in entries:
                check_logits(got[at : at + n], want[i][s : s + n], dtype, f"{name} request {i} tokens {s}..{s + n}")
                at += n
        assert rp.close() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(TINY))
def test_first_tokens_one_by_one(name, dtype, folders, truth, tmp_path):
    """A sequence fed one token at a time from its very first token: positions 0, 1, 2, ... on the
    decode path, four sequences side by side."""
    reqs, want = truth[name]
    picked = [i for i in range(len(reqs)) if len(reqs[i]) >= 20][:4]
    with Replay(folders[name], dtype, tmp_path / "out", 64 * len(picked)) as rp:
        for p in range(20):
            got = rp.step([(f"r{i}", [reqs[i][p]], [0]) for i in picked], end=[f"r{i}" for i in picked] if p == 19 else [])
            for k, i in enumerate(picked):
                check_logits(got[k : k + 1], want[i][p : p + 1], dtype, f"{name} request {i} position {p}")
        assert rp.close() == 0
