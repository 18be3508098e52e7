"""The host's plan for handing the keys of deep prefill tiles out in parts: every key tile of every
tile is visited exactly once, parts of a tile lie in consecutive slots in ascending key order, and
batches whose whole tiles already balance are left alone."""

from __future__ import annotations

import random

import pytest

from miniserve_amd.kernels.ops import PREFILL_KEY_TILE, PREFILL_MIN_PART, plan_prefill_parts


def tiles_of(row_lens, row_starts, tile_tokens):
    out, t = [], 0
    for n, s in zip(row_lens, row_starts):
        if n > 1:
            for a in range(0, n, tile_tokens):
                c = min(tile_tokens, n - a)
                out.append((t + a, c, (s + a + c - 1) // PREFILL_KEY_TILE + 1))
        t += n
    return out


@pytest.mark.parametrize("seed", range(30))
def test_parts_cover_every_key_tile_once(seed):
    rng = random.Random(seed)
    rows = rng.randint(1, 5)
    lens = [rng.choice([1, 2, 31, 64, 200, 700, 2048]) for _ in range(rows)]
    starts = [rng.choice([0, 5, 63, 64, 1000, 5000]) for _ in range(rows)]
    tile_tokens, kv_heads = rng.choice([8, 16, 32, 64, 128]), rng.choice([1, 2, 8])
    plan = plan_prefill_parts(lens, starts, tile_tokens, kv_heads)
    if plan is None:
        return
    entries, merges = plan
    want = {(f, c): d for f, c, d in tiles_of(lens, starts, tile_tokens)}
    seen = {}
    for first, count, kb, ke, slot in entries:
        assert 0 <= kb < ke <= want[(first, count)], "a part is empty or reaches past the tile's last key tile"
        seen.setdefault((first, count), []).append((kb, ke, slot))
    assert set(seen) == set(want), "every tile has an entry"
    weights = [ke - kb for _, _, kb, ke, _ in entries]
    assert weights == sorted(weights, reverse=True), "heaviest entries first"
    merged = {(f, c): (s0, n) for f, c, s0, n in merges}
    slots = []
    for key, parts in seen.items():
        parts.sort()
        assert parts[0][0] == 0 and parts[-1][1] == want[key]
        assert all(a[1] == b[0] for a, b in zip(parts, parts[1:])), "parts follow each other without gap or overlap"
        if len(parts) == 1:
            assert parts[0][2] == -1 and key not in merged
        else:
            s0, n = merged[key]
            assert [p[2] for p in parts] == list(range(s0, s0 + n)), "ascending keys lie in consecutive slots"
            assert all(ke - kb >= 1 for kb, ke, _ in parts)
            slots += [p[2] for p in parts]
    assert sorted(slots) == list(range(len(slots))), "slots are used once each, without holes"


def test_only_a_chain_much_longer_than_the_chip_is_busy_is_cut():
    # A 512-token portion behind 16,000 cached tokens, 32 tokens per tile, 8 KV heads: 128 blocks that
    # each walk about 256 key tiles; the fair share is 64 key tiles.
    entries, merges = plan_prefill_parts([512], [16000], 32, 8)
    assert max(ke - kb for _, _, kb, ke, _ in entries) <= 66 and len(merges) == 16
    assert all(n >= 4 for _, _, _, n in merges)
    # One 2,048-token prompt: the deepest chain (32) is no longer than the chip is busy anyway.
    assert plan_prefill_parts([2048], [0], 32, 8) is None
    assert plan_prefill_parts([1024], [0], 32, 8) is None
    assert plan_prefill_parts([2048] * 4, [0] * 4, 32, 8) is None  # 2,048 blocks: whole tiles balance
    assert plan_prefill_parts([100], [0], 32, 8) is None  # no tile deeper than the shortest part
    assert plan_prefill_parts([1, 1, 1], [5, 6, 7], 32, 8) is None  # no tile at all
    # A portion of 200 tokens beside decode rows, 8,000 tokens into its sequence: cut.
    assert plan_prefill_parts([1, 200, 1], [100, 8000, 7], 32, 8) is not None
    assert PREFILL_MIN_PART >= 1
