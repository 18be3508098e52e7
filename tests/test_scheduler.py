"""The scheduler's decisions and the engine loop on the CPU, with the real cache manager under a
toy runner. Exact (request, start, new tokens) rows per step for the reference's cases
(tests/test_engine.py:141-202,286-345,355-408), then random load under page pressure: every request
produces what it produces alone, pages never leak, budgets hold."""

import random

import pytest

from miniserve_amd.engine.engine import Engine
from miniserve_amd.engine.request import InvalidTransition, Request, RequestState, SamplingParams
from miniserve_amd.engine.scheduler import Phase, Scheduler
from toy_runner import ToyRunner, ToySampler, run_alone


def req(rid, n, new=8):
    return Request(rid, list(range(1, n + 1)), SamplingParams(new))


def sched(pages, chunk=0, **kw):
    runner = ToyRunner(pages, page_size=4, **{k: v for k, v in kw.items() if k in ("windows", "max_step_tokens")})
    s = Scheduler(cache=runner.cache, chunked_prefill_size=chunk,
                  **{k: v for k, v in kw.items() if k in ("max_running", "max_prefill_tokens")})
    return s, runner


def run(batch, runner):
    """What the engine does with a batch, with token 0 as every sampled token."""
    from miniserve_amd.engine.batch import StepRow

    done = batch.completes()
    runner.step([StepRow(r.cache, r.step_tokens(s, n)[0], [n - 1] if d else [])
                 for (r, s, n), d in zip(batch.rows, done)])
    for r, d in zip(batch.requests, done):
        if d:
            r.sampled(0)
            r.read_back(0)
            if r.state is RequestState.PREFILL:
                r.transition(RequestState.DECODE)


def rows(b):
    return [(r.rid, s, n) for r, s, n in zip(b.requests, b.starts, b.extend_lens)]


# ------------------------------------------------------------------------------------------ requests


def test_state_machine():
    r = req(0, 3)
    with pytest.raises(InvalidTransition):
        r.transition(RequestState.DECODE)
    r.transition(RequestState.PREFILL)
    r.transition(RequestState.WAITING)  # preempted between portions
    r.transition(RequestState.PREFILL)
    r.transition(RequestState.FINISHED)  # straight from prefill
    assert r.is_done
    with pytest.raises(InvalidTransition):
        r.transition(RequestState.WAITING)
    with pytest.raises(ValueError):
        Request(1, [], SamplingParams(1))


def test_sampling_params_are_checked():
    for kw in (dict(max_new_tokens=0), dict(max_new_tokens=1, temperature=-1), dict(max_new_tokens=1, top_p=0),
               dict(max_new_tokens=1, top_p=1.5), dict(max_new_tokens=1, seed=2**32), dict(max_new_tokens=1, seed=-1)):
        with pytest.raises(ValueError):
            SamplingParams(**kw)
    assert SamplingParams(1).is_greedy and not SamplingParams(1, temperature=0.5).is_greedy


def test_step_tokens_span_prompt_and_output_and_name_what_is_in_flight():
    r = req(0, 4)
    for tok in (9, 8, 7):
        r.sampled(0)
        assert not r.read_back(tok)
    assert r.prompt_ids == [1, 2, 3, 4] and r.output_ids == [9, 8, 7]
    assert r.step_tokens(0, 4) == ([1, 2, 3, 4], None) and r.step_tokens(2, 4) == ([3, 4, 9, 8], None)
    assert r.step_tokens(5, 2) == ([8, 7], None) and r.seq_len == 7 and r.max_len == 12
    r.sampled(5)  # the next token lies at index 5 of the latest step's sampled tokens, not yet on the host
    assert r.seq_len == 8 and r.num_output == 4 and r.output_ids == [9, 8, 7]
    assert r.step_tokens(7, 1) == ([0], 5) and r.step_tokens(5, 3) == ([8, 7, 0], 5) and r.step_tokens(5, 2) == ([8, 7], None)
    with pytest.raises(RuntimeError):
        r.step_tokens(7, 2)
    r.sampled(2)  # launched once more before the read-back
    assert r.seq_len == 9 and r.read_back(6) is False and r.seq_len == 9 and r.in_flight == 1 and r.feed == 2
    short = Request(1, [5], SamplingParams(2, stop_token_ids={3}))
    short.sampled(0)
    assert not short.sampled_all and short.read_back(3) and short.forget_in_flight() == 0  # the stop token ends it and is kept
    assert short.output_ids == [3]


# ------------------------------------------------------------------------------------------ whole prefills


def test_prefill_first_then_decode():
    s, runner = sched(64)
    a, b = req(0, 3), req(1, 5)
    s.add(a); s.add(b)
    batch = s.schedule()
    assert batch.phase is Phase.PREFILL and rows(batch) == [(0, 0, 3), (1, 0, 5)]
    run(batch, runner)
    batch = s.schedule()
    assert batch.phase is Phase.DECODE and rows(batch) == [(0, 3, 1), (1, 5, 1)]
    c = req(2, 2)
    s.add(c)
    batch = s.schedule()  # a new arrival goes before the decode step
    assert batch.phase is Phase.PREFILL and batch.requests == [c]
    run(batch, runner)
    assert s.schedule().requests == [a, b, c]


def test_prefill_token_budget_and_oversized_prompt():
    s, _ = sched(64, max_prefill_tokens=10)
    rs = [req(i, 4) for i in range(4)]
    for r in rs:
        s.add(r)
    assert s.schedule().requests == rs[:2] and s.schedule().requests == rs[2:]
    s, _ = sched(64, max_prefill_tokens=10)
    big, small = req(0, 50), req(1, 2)
    s.add(big); s.add(small)
    assert s.schedule().requests == [big] and s.schedule().requests == [small]


def test_max_running_and_retire():
    s, runner = sched(64, max_running=2)
    rs = [req(i, 1) for i in range(3)]
    for r in rs:
        s.add(r)
    batch = s.schedule()
    assert batch.requests == rs[:2]
    run(batch, runner)
    assert s.schedule().phase is Phase.DECODE
    with pytest.raises(ValueError):
        s.retire(rs[0])
    rs[0].transition(RequestState.FINISHED)
    runner.release(rs[0].cache)
    s.retire(rs[0])
    assert s.schedule().requests == [rs[2]]


def test_admission_reserves_prefill_and_next_token():
    s, _ = sched(3)
    x, y = req(0, 4), req(1, 4)  # each needs ceil((4 + 1) / 4) = 2 pages
    s.add(x); s.add(y)
    assert s.schedule().requests == [x]
    assert y.cache is None and list(s.waiting) == [y]  # the refused admission left nothing behind


def test_admission_keeps_room_for_running_decodes_and_does_not_skip_ahead():
    s, runner = sched(4)
    x = req(0, 8)
    s.add(x)
    run(s.schedule(), runner)
    big, small = req(1, 4), req(2, 2)
    s.add(big); s.add(small)
    batch = s.schedule()
    assert batch.phase is Phase.DECODE and batch.requests == [x] and not batch.preempted
    assert list(s.waiting) == [big, small] and runner.cache.state_slots.num_free == runner.cache.state_slots.num_slots - 1


def test_preemption_newest_first_back_to_front_of_queue():
    s, runner = sched(6)
    x, y, z = (req(i, 4, 20) for i in range(3))
    for r in (x, y, z):
        s.add(r)
    run(s.schedule(), runner)
    late = req(3, 4, 20)
    s.add(late)
    for _ in range(4):
        batch = s.schedule()
        assert batch.phase is Phase.DECODE and not batch.preempted
        run(batch, runner)
    assert runner.cache.free_pages() == [0]
    batch = s.schedule()
    assert batch.requests == [x, y] and batch.preempted == [z]
    assert z.state is RequestState.WAITING and z.cache is None and z.num_preemptions == 1
    assert list(s.waiting) == [z, late] and s.running == [x, y] and s.num_preemptions == 1
    assert z.seq_len == 4 + 5  # it resumes with its output kept
    run(batch, runner)
    runner.cache.check_invariants()


def test_lone_request_is_never_preempted_and_too_large_is_refused():
    s, runner = sched(3)
    x = req(0, 4, 8)
    s.add(x)
    while not x.sampled_all:
        batch = s.schedule()
        assert not batch.preempted
        run(batch, runner)
    assert runner.cache.free_pages() == [0]
    s, _ = sched(3)
    with pytest.raises(ValueError, match="pool holds"):
        s.add(req(0, 10, 3))
    s.add(req(1, 10, 2))


# ------------------------------------------------------------------------------------------ portions


def test_chunked_decode_first_then_portions():
    s, runner = sched(64, chunk=8)
    x = req(0, 3)
    s.add(x)
    b = s.schedule()
    assert b.phase is Phase.PREFILL and rows(b) == [(0, 0, 3)]
    run(b, runner)
    long = req(1, 20, 4)
    s.add(long)
    b = s.schedule()
    assert b.phase is Phase.MIXED and rows(b) == [(0, 3, 1), (1, 0, 7)] and b.completes() == [True, False] and b.num_decode == 1
    run(b, runner)
    assert long.state is RequestState.PREFILL and long.output_ids == [] and long.cache.num_tokens == 7
    b = s.schedule()
    assert rows(b) == [(0, 4, 1), (1, 7, 7)]
    run(b, runner)
    b = s.schedule()
    assert rows(b) == [(0, 5, 1), (1, 14, 6)] and b.completes() == [True, True]
    run(b, runner)
    assert long.state is RequestState.DECODE and long.output_ids == [0]
    b = s.schedule()
    assert b.phase is Phase.DECODE and rows(b) == [(0, 6, 1), (1, 20, 1)]


def test_chunked_budget_counts_decodes_and_admits_in_order():
    s, runner = sched(64, chunk=6)
    xs = [req(i, 2) for i in range(3)]
    for x in xs:
        s.add(x)
    b = s.schedule()
    assert rows(b) == [(0, 0, 2), (1, 0, 2), (2, 0, 2)]
    run(b, runner)
    y, z = req(3, 10, 4), req(4, 1, 4)
    s.add(y); s.add(z)
    b = s.schedule()
    assert rows(b) == [(0, 2, 1), (1, 2, 1), (2, 2, 1), (3, 0, 3)] and list(s.waiting) == [z] and b.num_tokens == 6


def test_chunked_admission_reserves_whole_prefill():
    s, runner = sched(6, chunk=4)
    x, y = req(0, 16, 4), req(1, 4, 4)  # x needs ceil(17 / 4) = 5 pages, y 2
    s.add(x); s.add(y)
    b = s.schedule()
    assert rows(b) == [(0, 0, 4)]
    run(b, runner)
    b = s.schedule()
    assert rows(b) == [(0, 4, 4)] and list(s.waiting) == [y]


def test_chunked_preempts_newest_even_mid_prefill():
    s, runner = sched(8, chunk=4)
    x = req(0, 4, 28)
    s.add(x)
    run(s.schedule(), runner)
    y = req(1, 20, 4)
    s.add(y)
    for step in range(4):
        b = s.schedule()
        assert rows(b) == [(0, 4 + step, 1), (1, 3 * step, 3)] and not b.preempted
        run(b, runner)
    assert x.cache.num_tokens == 8 and y.cache.num_tokens == 12 and y.state is RequestState.PREFILL
    b = s.schedule()  # x's next token needs a third page; y's reservation leaves none
    assert b.preempted == [y] and y.state is RequestState.WAITING and y.cache is None
    assert b.phase is Phase.DECODE and rows(b) == [(0, 8, 1)]
    run(b, runner)
    assert list(s.waiting) == [y] and y.num_preemptions == 1
    runner.cache.check_invariants()


def test_whole_prompt_above_the_budget_holds_all_its_tokens_in_a_windowed_group():
    """Whole prompts run in one step whatever the prefill budget, so a windowed group holds the whole
    prompt for that step: admission and the refusal at submission count it so, and the step fits."""
    s, runner = sched(10, chunk=0, windows=(6,), max_prefill_tokens=8)
    with pytest.raises(ValueError, match="pool holds"):
        s.add(req(9, 40, 2))  # 11 pages in one step although the window is 6
    a, b = req(0, 26, 3), req(1, 26, 3)  # ceil(27 / 4) = 7 pages for the prefill step, then 2-3 behind the window
    s.add(a); s.add(b)
    batch = s.schedule()
    assert rows(batch) == [(0, 0, 26)] and list(s.waiting) == [b]  # b's prompt does not fit beside a's
    run(batch, runner)
    assert a.cache.tables[0].num_held <= 3 and runner.cache.free_pages() == [10 - a.cache.tables[0].num_held]
    batch = s.schedule()  # now that the window has passed most of a's pages, b is let in: alone, before a decodes
    assert rows(batch) == [(1, 0, 26)] and not batch.preempted
    run(batch, runner)
    assert rows(s.schedule()) == [(0, 26, 1), (1, 26, 1)]
    runner.cache.check_invariants()


def test_requests_whose_tokens_are_all_sampled_hold_nothing():
    """With the read-back one step behind, a request whose last token has been sampled gives its pages
    back at that launch. Two requests fill a pool of 4 pages; the older one still decodes and needs a
    page for its next token when the newer one has just sampled its last: nobody is preempted."""
    eng = toy_engine(4, 0, overlap=True)
    a = eng.add_request([1, 2, 3, 4, 5, 6, 7], SamplingParams(6))
    b = eng.add_request([1, 2, 3, 4, 5, 6], SamplingParams(2))
    eng.step()  # both prompts: 2 pages each, the pool is full
    assert eng.runner.cache.free_pages() == [0]
    eng.step()  # first decode step: a's 8th token fits its page; b samples its last token and lets go
    assert b.cache is None and b.in_flight == 1 and not b.is_done and eng.runner.cache.free_pages() == [2]
    while eng.has_unfinished:
        eng.step()
        eng.runner.cache.check_invariants()
    assert eng.scheduler.num_preemptions == 0 and eng.runner.cache.idle
    assert len(a.output_ids) == 6 and len(b.output_ids) == 2


def test_windowed_groups_let_more_requests_in():
    """With a window of 8 the windowed group never holds more than the window plus one step, so a
    long request needs far fewer pages there than its length."""
    s, runner = sched(8, chunk=4, windows=(8,), max_step_tokens=4)
    a, b = req(0, 60, 2), req(1, 60, 2)  # 16 pages each if all keys were kept: would be refused
    s.add(a); s.add(b)
    batch = s.schedule()
    assert rows(batch) == [(0, 0, 4)]
    while s.has_unfinished and (batch := s.schedule()) is not None:
        run(batch, runner)
        for r in list(batch.requests):
            if r.sampled_all and r.state is RequestState.DECODE:
                r.transition(RequestState.FINISHED)
                runner.release(r.cache)
                s.retire(r)
        assert max(t.num_held for r in s.running for t in r.cache.tables) <= 4 if s.running else True
    assert a.is_done and b.is_done and runner.cache.idle


# ------------------------------------------------------------------------------------------ the loop under load


def toy_engine(pages, chunk, windows=(0,), max_running=8, backend="python", seed=0, overlap=True, max_prefill_tokens=64):
    runner = ToyRunner(pages, page_size=4, windows=windows, max_running=max_running, max_step_tokens=chunk or None, backend=backend)
    return Engine(None, max_running=max_running, max_prefill_tokens=max_prefill_tokens, runner=runner, chunked_prefill_size=chunk,
                  seed=seed, sampler=ToySampler(), overlap=overlap)


@pytest.mark.parametrize("overlap", [True, False])
@pytest.mark.parametrize("pages,chunk,windows,backend", [
    (8, 3, (0,), "python"), (16, 0, (0,), "cpp"), (64, 2048, (0,), "python"), (8, 5, (0, 6), "cpp"), (12, 7, (10,), "python"),
    (10, 0, (0,), "python"), (10, 0, (6,), "cpp"), (10, 0, (0, 6), "python"),
])
def test_load_under_page_pressure(pages, chunk, windows, backend, overlap):
    """As the reference's load test (tests/test_engine.py:562-598): random requests and arrivals, pools
    that force preemption, whole and chunked prefill, the read-back one step behind or not; every
    output equals the request's run alone. The pools of 10 pages run whole prompts of up to 30 tokens
    under a prefill budget of 8 (a prompt above the budget is admitted alone and must hold all its
    tokens in that one step, window or not) and new tokens up to what the pool holds."""
    preemptions = 0
    for seed in range(10 if pages == 10 else 6):
        preemptions += _load(seed, pages, chunk, windows, backend, overlap)
    if pages <= 10:
        assert preemptions > 0, "the small pool was meant to force preemption"


def _load(seed, pages, chunk, windows, backend, overlap=True) -> int:
    rng = random.Random(seed)
    tight = pages == 10
    eng = toy_engine(pages, chunk, windows, backend=backend, seed=seed, overlap=overlap, max_prefill_tokens=8 if tight else 64)
    vocab = eng.runner.model.vocab_size
    submitted = []
    pending = []
    for i in range(40):
        n, new = (rng.randint(1, 30), rng.randint(1, 10)) if tight else (rng.randint(1, 12), rng.randint(1, 16))
        kind = rng.choice(("greedy", "hot", "nucleus"))
        sp = SamplingParams(new, stop_token_ids=frozenset({rng.randrange(vocab)}) if rng.random() < 0.3 else frozenset(),
                            temperature=0.0 if kind == "greedy" else 4.0, top_p=0.9 if kind == "nucleus" else 1.0,
                            seed=rng.randrange(2**32) if rng.random() < 0.5 else None)
        pending.append((rng.randint(0, 30), [rng.randrange(vocab) for _ in range(n)], sp))
    pending.sort(key=lambda t: t[0])
    step = 0
    while pending or eng.has_unfinished:
        while pending and pending[0][0] <= step:
            _, prompt, sp = pending.pop(0)
            submitted.append(eng.add_request(prompt, sp))
        batch = eng.step()
        step += 1
        eng.runner.cache.check_invariants()
        if batch is not None and chunk:
            assert batch.num_tokens <= chunk
        assert step < 5000, "the engine stalls"
    assert eng.runner.cache.idle, "pages or state slots leaked"
    for r in submitted:
        assert r.state is RequestState.FINISHED
        assert r.output_ids == run_alone(r.prompt_ids, r.params, r.seed, vocab), f"request {r.rid} differs from its run alone"
    return eng.scheduler.num_preemptions


def test_engine_assigns_seeds_in_submission_order():
    a, b = toy_engine(64, 8, seed=5), toy_engine(64, 8, seed=5)
    sp = SamplingParams(4, temperature=1.0)
    ra = [a.add_request([1, 2, 3], sp) for _ in range(3)]
    rb = [b.add_request([1, 2, 3], sp) for _ in range(3)]
    assert [r.seed for r in ra] == [r.seed for r in rb] and len({r.seed for r in ra}) == 3
    assert a.add_request([1], SamplingParams(1, seed=77)).seed == 77


def test_overlap_drops_what_runs_past_a_stop():
    """With the read-back one step behind, a request that samples its stop token has already been
    launched once more: that token is dropped and the outputs are what the synchronous loop gives.
    (The reference counts the same cases, tests/test_engine.py:601-641.)"""
    dropped = 0
    for seed in range(12):
        outs = []
        for overlap in (True, False):
            rng = random.Random(seed)
            eng = toy_engine(8, 3, seed=seed, overlap=overlap)
            vocab = eng.runner.model.vocab_size
            reqs = [eng.add_request([rng.randrange(vocab) for _ in range(rng.randint(1, 9))],
                                    SamplingParams(rng.randint(1, 14), temperature=4.0, seed=rng.randrange(2**32),
                                                   stop_token_ids=frozenset(rng.sample(range(vocab), 8))))
                    for _ in range(12)]
            steps = 0
            while eng.has_unfinished:
                eng.step()
                eng.runner.cache.check_invariants()
                steps += 1
                assert steps < 3000
            assert eng.runner.cache.idle and all(r.in_flight == 0 for r in reqs)
            outs.append([r.output_ids for r in reqs])
            if overlap:
                dropped += eng.dropped_tokens
            else:
                assert eng.dropped_tokens == 0
        assert outs[0] == outs[1]
    assert dropped > 0, "no request ran past its stop token: the case was meant to occur"


def test_overlap_request_ends_while_it_waits_after_a_preemption(monkeypatch):
    """Two requests of 7 tokens in a pool of 4 pages of 4: both decode until each needs a third page, and
    the newer one is preempted, while the token of its last step is still on its way. That token is its
    stop token: it ends from WAITING, and never runs again."""
    seen = []
    plain_transition = Request.transition

    def recording(self, new):
        seen.append((self.rid, self.state, new))
        plain_transition(self, new)

    monkeypatch.setattr(Request, "transition", recording)
    vocab, prompt_a, prompt_b = 50, [3, 1, 4, 1, 5, 9, 2], [2, 7, 1, 8, 2, 8, 1]
    alone = run_alone(prompt_b, SamplingParams(9), 5, vocab)
    assert alone[0] != alone[1], "the second token was meant to be the first stop"
    eng = toy_engine(4, 16, seed=0, overlap=True)
    a = eng.add_request(prompt_a, SamplingParams(9, seed=4))
    b = eng.add_request(prompt_b, SamplingParams(9, seed=5, stop_token_ids=frozenset({alone[1]})))
    while eng.has_unfinished:
        eng.step()
        eng.runner.cache.check_invariants()
    assert b.output_ids == alone[:2] and a.output_ids == run_alone(prompt_a, a.params, 4, vocab)
    assert (b.rid, RequestState.DECODE, RequestState.WAITING) in seen, "the newer request was meant to be preempted"
    assert (b.rid, RequestState.WAITING, RequestState.FINISHED) in seen
    assert eng.scheduler.num_preemptions == 1 and eng.runner.cache.idle


@pytest.mark.parametrize("overlap", [True, False])
def test_abort_at_any_time_returns_everything(overlap):
    for at in range(0, 12, 2):
        eng = toy_engine(16, 4, overlap=overlap)
        rs = [eng.add_request(list(range(1, 10)), SamplingParams(10)) for _ in range(3)]
        for _ in range(at):
            eng.step()
        eng.abort(rs[1].rid)
        eng.abort(rs[1].rid)
        eng.abort(999)
        while eng.has_unfinished:
            eng.step()
        assert rs[1].state is RequestState.ABORTED and rs[0].state is RequestState.FINISHED
        assert eng.runner.cache.idle and not eng.requests


def test_refused_at_submission_what_could_never_run():
    runner = ToyRunner(64, page_size=4)
    s = Scheduler(cache=runner.cache, chunked_prefill_size=0, max_step_tokens=20, max_prefill_tokens=16, max_position=40)
    with pytest.raises(ValueError, match="max_position_embeddings"):
        s.add(req(0, 38, 3))  # 41 tokens at most
    s.add(req(1, 18, 3))
    with pytest.raises(ValueError, match="chunked prefill"):
        s.add(req(2, 22, 2))  # prefilled again after a preemption it would run 23 tokens in one step
    chunked = Scheduler(cache=runner.cache, chunked_prefill_size=8, max_step_tokens=20, max_position=40)
    chunked.add(req(3, 30, 2))  # portions of 8 fit any step
    with pytest.raises(ValueError, match="at most 20"):
        Scheduler(cache=runner.cache, chunked_prefill_size=32, max_step_tokens=20)
    with pytest.raises(ValueError, match="at most 20"):
        Scheduler(cache=runner.cache, chunked_prefill_size=0, max_prefill_tokens=64, max_step_tokens=20)
