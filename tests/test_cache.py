"""The cache manager on the CPU: allocator, tables and packing in both implementations (Python and
C++), checked against the reference's vectors (tests/test_block_allocator.py:50-58,146-177,200-217)
and against each other; groups, windows and state slots; and under random orders of requests: no
page lost, held twice or freed twice."""

import random

import numpy as np
import pytest

from miniserve_amd.cache import NO_PAGE, PageAllocator, CacheLayout, CacheManager, OutOfBlocks, OutOfStateSlots, pack_tables
from miniserve_amd.cache.backend import allocator_class
from miniserve_amd.cache.native import NativePageAllocator
from miniserve_amd.parts.base import CachePlane, KVNeed, StateNeed, StateTensor
from miniserve_amd.parts.model import CacheSlotNeed

BACKENDS = [PageAllocator, NativePageAllocator]


@pytest.mark.parametrize("A", BACKENDS)
def test_allocation_order_is_part_of_the_contract(A):
    a = A(8, 4)
    assert a.take(3) == [0, 1, 2] and a.take(2) == [3, 4]
    a.give_back([1, 3])
    assert a.take(1) == [3] and a.take(3) == [1, 5, 6]
    assert a.num_free == 1 and a.num_used == 7
    a.check_invariants()


@pytest.mark.parametrize("A", BACKENDS)
def test_allocate_is_all_or_nothing_and_free_checks_first(A):
    a = A(4, 2)
    got = a.take(3)
    with pytest.raises(OutOfBlocks):
        a.take(2)
    assert a.num_free == 1
    with pytest.raises(ValueError):
        a.give_back([got[0], got[0]])  # one holder, two releases
    with pytest.raises(IndexError):
        a.give_back([got[0], 99])
    assert a.holders_of(got[0]) == 1 and a.num_free == 1  # nothing changed
    a.hold([got[0]])
    a.give_back([got[0], got[0]])
    assert a.holders_of(got[0]) == 0
    with pytest.raises(ValueError):
        a.hold([got[0]])  # a free block
    with pytest.raises(ValueError):
        A(0, 4)
    a.check_invariants()


@pytest.mark.parametrize("A", BACKENDS)
def test_table_vectors(A):
    a = A(8, 4)
    t = a.new_table()
    assert t.append(5) == [0, 1] and t.pages == [0, 1]
    assert [t.slot(p) for p in range(5)] == [0, 1, 2, 3, 4]
    assert t.append(3) == [] and t.append(1) == [2] and t.slot(8) == 8
    assert [t.pages_needed(n) for n in (0, 3, 4, 8)] == [0, 0, 1, 2]
    with pytest.raises(IndexError):
        t.slot(9)
    a2 = A(8, 4)
    a2.take(4)
    a2.give_back([1, 3])
    t2 = a2.new_table()
    t2.append(6)
    assert t2.pages == [3, 1] and t2.tail_slots(6) == [12, 13, 14, 15, 4, 5] and t2.tail_slots(2) == [4, 5]
    t2.rewind(3)  # keeps its blocks: recomputed tokens land in the same slots
    assert t2.num_tokens == 3 and t2.pages == [3, 1] and t2.pages_needed(5) == 0
    t2.release()
    assert t2.pages == [] and a2.num_free == 6
    with pytest.raises(OutOfBlocks):
        A(2, 4).new_table().append(9)


@pytest.mark.parametrize("A", BACKENDS)
def test_shared_prefix(A):
    a = A(8, 4)
    first = a.new_table()
    first.append(8)
    second = a.new_table(first.pages)
    assert second.num_tokens == 8 and a.holders_of(0) == 2
    assert second.append(1) == [2]  # new tokens go to a block of its own
    first.release()
    assert a.holders_of(0) == 1 and a.num_free == 5
    second.release()
    assert a.num_free == 8
    with pytest.raises(ValueError, match="duplicate"):
        a.new_table([1, 1])


@pytest.mark.parametrize("A", BACKENDS)
def test_release_before_gives_back_whole_pages_only(A):
    a = A(8, 4)
    t = a.new_table()
    t.append(14)
    assert t.release_before(3) == 0
    assert t.release_before(9) == 2 and t.pages == [NO_PAGE, NO_PAGE, 2, 3] and t.num_held == 2
    assert a.num_free == 6 and t.release_before(9) == 0
    assert t.tail_slots(6) == [8, 9, 10, 11, 12, 13]
    with pytest.raises(IndexError):
        t.slot(7)
    with pytest.raises(IndexError):
        t.tail_slots(7)
    assert t.append(3) == [1]  # the newest freed page comes back first
    t.release()
    assert a.num_free == 8
    a.check_invariants()


@pytest.mark.parametrize("A", BACKENDS)
def test_packing_is_the_naive_dense_layout(A):
    a = A(16, 4)
    tables = []
    for n in (5, 0, 13):
        t = a.new_table()
        t.append(n)
        tables.append(t)
    tables[2].release_before(6)
    out = np.full((5, 6), 77, dtype=np.int32)
    assert pack_tables(tables, out, pad_rows=2, pad_page=9) == 6
    want = [[0, 1, 9, 9, 9, 9], [9] * 6, [NO_PAGE, 3, 4, 5, 9, 9], [9] * 6, [9] * 6]
    assert out.tolist() == want
    with pytest.raises(ValueError):
        pack_tables(tables, np.zeros((3, 3), dtype=np.int32))
    with pytest.raises(ValueError):
        pack_tables(tables, np.zeros((2, 6), dtype=np.int32))


def test_backends_agree_under_random_operations():
    for seed in range(10):
        rng = random.Random(seed)
        py, cc = PageAllocator(24, 4), NativePageAllocator(24, 4)
        tp, tc = [], []
        for _ in range(300):
            op = rng.random()
            if op < 0.35 or not tp:
                tp.append(py.new_table()); tc.append(cc.new_table())
            i = rng.randrange(len(tp))
            if op < 0.7:
                n = rng.randrange(0, 11)
                try:
                    got = tp[i].append(n)
                except OutOfBlocks:
                    with pytest.raises(OutOfBlocks):
                        tc[i].append(n)
                else:
                    assert tc[i].append(n) == got
            elif op < 0.85:
                pos = rng.randrange(0, tp[i].num_tokens + 1)
                assert tp[i].release_before(pos) == tc[i].release_before(pos)
            else:
                tp.pop(i).release(); tc.pop(i).release()
            assert py.num_free == cc.num_free
            for a, b in zip(tp, tc):
                assert a.pages == b.pages and a.num_tokens == b.num_tokens and a.num_held == b.num_held
            py.check_invariants(); cc.check_invariants()


# ------------------------------------------------------------------------------------------ manager


def layout(windows=(0, 0, 8), state=False):
    needs = [CacheSlotNeed(i, KVNeed.keys_values(2, 16, w), StateNeed.single((3,)) if state and i == 0 else None)
             for i, w in enumerate(windows)]
    return CacheLayout.from_needs(needs)


def test_layers_are_grouped_by_their_needs():
    lay = CacheLayout.from_needs([
        CacheSlotNeed(0, KVNeed.keys_values(2, 16, 8), None), CacheSlotNeed(1, KVNeed.keys_values(2, 16, 0), None),
        CacheSlotNeed(2, KVNeed.keys_values(2, 16, 8), None), CacheSlotNeed(3, KVNeed.keys_values(1, 32, 0), StateNeed.single((4, 2))),
        CacheSlotNeed(4, None, StateNeed((StateTensor("sum", (5,)), StateTensor("seen", (1,), "int32")))),
    ])
    assert [(g.planes[0].heads, g.planes[0].width, g.window, g.slots) for g in lay.groups] == [
        (1, 32, 0, (3,)), (2, 16, 0, (1,)), (2, 16, 8, (0, 2))]
    assert all([p.name for p in g.planes] == ["k", "v"] and g.planes[1].token_minor and not g.planes[0].token_minor for g in lay.groups)
    assert [(s.slot, [(t.name, t.shape, t.dtype) for t in s.tensors]) for s in lay.states] == [
        (3, [("state", (4, 2), "float32")]), (4, [("sum", (5,), "float32"), ("seen", (1,), "int32")])]
    assert lay.bytes_per_page(16, 2) == [2 * 1 * 16 * 32 * 2, 2 * 1 * 16 * 32 * 2, 2 * 2 * 16 * 32 * 2]


def test_the_pool_is_built_from_what_the_mixers_say_they_keep():
    """A mixer names its per-token record as planes: keys and values of different widths, or one latent
    vector per token, get pages of their own shape without a change to the pool; state may be several
    tensors of different dtypes."""
    import torch

    from miniserve_amd.cache.pool import KVPool

    lay = CacheLayout.from_needs([
        CacheSlotNeed(0, KVNeed((CachePlane("k", 2, 32), CachePlane("v", 2, 16, token_minor=True)), 0), None),
        CacheSlotNeed(1, KVNeed((CachePlane("latent", 1, 24),), 0), StateNeed((StateTensor("sum", (6,)), StateTensor("seen", (1,), "int32")))),
        CacheSlotNeed(2, KVNeed((CachePlane("latent", 1, 24),), 0), None),
    ])
    assert [[p.name for p in g.planes] for g in lay.groups] == [["k", "v"], ["latent"]] and lay.groups[1].slots == (1, 2)
    assert lay.bytes_per_page(4, 2) == [1 * 4 * (2 * 32 + 2 * 16) * 2, 2 * 4 * 24 * 2]
    pool = KVPool(lay, 4, [5, 7], 3, torch.bfloat16, "cpu")
    assert tuple(pool.buffers[0]["k"].shape) == (1, 6, 2, 4, 32) and tuple(pool.buffers[0]["v"].shape) == (1, 6, 2, 16, 4)
    assert tuple(pool.buffers[1]["latent"].shape) == (2, 8, 1, 4, 24)
    assert pool.bytes_per_token() == (96 + 2 * 24) * 2 and pool.dummy_page(1) == 7
    state = pool.state_view(1, None)
    assert tuple(state["sum"].shape) == (4, 6) and state["sum"].dtype == torch.float32
    assert tuple(state["seen"].shape) == (4, 1) and state["seen"].dtype == torch.int32 and pool.state_view(0, None) is None
    with pytest.raises(ValueError, match="distinct names"):
        KVNeed((CachePlane("k", 1, 8), CachePlane("k", 1, 8)))
    with pytest.raises(ValueError, match="distinct names"):
        StateNeed(())


@pytest.mark.parametrize("backend", ["python", "cpp"])
def test_extend_is_all_or_nothing_across_groups(backend):
    m = CacheManager(layout(), 4, [8, 3], 4, allocator_class=allocator_class(backend))
    rc = m.acquire()
    m.extend(rc, 10)
    assert [t.num_held for t in rc.tables] == [3, 3] and rc.num_tokens == 10
    with pytest.raises(OutOfBlocks):
        m.extend(rc, 4)  # the second group is exhausted; the first must not move
    assert [t.num_tokens for t in rc.tables] == [10, 10] and m.free_pages() == [5, 0]
    m.release(rc)
    assert m.idle
    with pytest.raises(RuntimeError):
        m.release(rc)  # a handle is released once


@pytest.mark.parametrize("backend", ["python", "cpp"])
def test_windowed_groups_give_pages_back_behind_the_window(backend):
    m = CacheManager(layout(), 4, [16, 16], 2, allocator_class=allocator_class(backend))
    rc = m.acquire()
    held = []
    for _ in range(10):
        m.extend(rc, 3)
        m.advance(rc)
        held.append([t.num_held for t in rc.tables])
    # window 8, page 4: after n tokens, keys before n - 7 are dead; whole pages before that go back
    assert [h[1] for h in held] == [1, 2, 3, 2, 2, 3, 3, 2, 2, 3] and held[-1][0] == 8
    full, win = rc.tables
    assert win.first_live == (30 - 8 + 1) // 4
    assert m.peak_pages(1000, 3) == [250, 4] and m.peak_pages(6, 3) == [2, 2]
    m.release(rc)
    assert m.idle


def test_state_slots_travel_with_the_request():
    m = CacheManager(layout(state=True), 4, [8, 8], 2)
    a, b = m.acquire(), m.acquire()
    assert {a.state_slot, b.state_slot} == {0, 1}
    with pytest.raises(OutOfStateSlots):
        m.acquire()
    freed = a.state_slot
    m.release(a)
    assert a.state_slot is None
    c = m.acquire()
    assert c.state_slot == freed  # the slot is used again
    with pytest.raises(ValueError, match="twice"):
        m.state_slots.release(1 - freed) or m.state_slots.release(1 - freed)
    m.state_slots.acquire()  # put the probed slot back under b's name
    m.release(b)
    m.release(c)
    assert m.idle
    m.check_invariants()


@pytest.mark.parametrize("backend", ["python", "cpp"])
@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_lose_no_page(backend, seed):
    rng = random.Random(seed)
    m = CacheManager(layout((0, 5, 0, 12)), 4, [20, 10, 10], 6, max_step_tokens=9, allocator_class=allocator_class(backend))
    live = []
    for _ in range(400):
        op = rng.random()
        if (op < 0.3 and len(live) < 6) or not live:
            live.append(m.acquire())
        elif op < 0.85:
            rc = rng.choice(live)
            n = rng.randrange(1, 10)
            before = [(t.num_tokens, t.pages) for t in rc.tables]
            if m.can_extend(rc, n):
                m.extend(rc, n)
                m.advance(rc)
            else:
                with pytest.raises(OutOfBlocks):
                    m.extend(rc, n)
                assert before == [(t.num_tokens, t.pages) for t in rc.tables]
        else:
            m.release(live.pop(rng.randrange(len(live))))
        m.check_invariants()
        # every page is held by exactly one table or free
        for g, alloc in enumerate(m.allocators):
            held = [b for rc in live for b in rc.tables[g].pages if b != NO_PAGE]
            assert len(held) == len(set(held)) == alloc.num_pages - alloc.num_free
            assert all(alloc.holders_of(b) == 1 for b in held)
        for rc in live:
            for g, t in zip(m.layout.groups, rc.tables):
                if g.window:
                    assert t.num_held <= m.peak_pages(rc.num_tokens, 9)[g.index]
    for rc in live:
        m.release(rc)
    assert m.idle
