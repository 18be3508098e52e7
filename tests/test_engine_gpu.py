"""Generation through the Python entry point and the command line against the plain
implementation: greedy tokens, long decoding, chunked and unchunked prefill, a pool so small that
requests are preempted and recomputed, sampled requests beside greedy ones."""

from __future__ import annotations

import json
import subprocess
import sys

import numpy as np
import pytest

from models import TINY, make_folder
from plain import qwen3_plain as P
from plain.model_folder import read_model_folder
from replay_util import ROOT

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_folder(root, name) for name in TINY}


def engine(folder, dtype="float32", **kw):
    from miniserve_amd.engine.engine import Engine
    from miniserve_amd.loading import load_model

    return Engine(load_model(folder, dtype, "cuda:0"), **kw)


def prompts_for(cfg, lens, seed=3):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in lens]


@pytest.mark.parametrize("name", sorted(TINY))
@pytest.mark.parametrize("chunk", [0, 16, 2048])
def test_greedy_generation_equals_plain(name, chunk, folders):
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders[name])
    prompts = prompts_for(cfg, [1, 9, 40, 17])
    want = [P.greedy(cfg, w, p, 16) for p in prompts]
    eng = engine(folders[name], kv_pool_tokens=512, max_running=4, chunked_prefill_size=chunk)
    got = eng.generate(prompts, SamplingParams(max_new_tokens=16))
    assert got == want
    assert eng.runner.cache.idle


def test_preemption_and_recompute_change_nothing(folders):
    """A pool that cannot hold all requests at once: some are preempted, prefilled again with
    their output kept, and still produce the tokens they produce alone."""
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders["tinyB"])
    prompts = prompts_for(cfg, [30, 45, 20, 38, 25, 41], seed=4)
    want = [P.greedy(cfg, w, p, 24) for p in prompts]
    eng = engine(folders["tinyB"], kv_pool_tokens=16 * 12, max_running=6, chunked_prefill_size=32)
    got = eng.generate(prompts, SamplingParams(max_new_tokens=24))
    assert eng.scheduler.num_preemptions > 0, "the pool was meant to be too small"
    assert got == want
    assert eng.runner.cache.idle


def test_long_decoding(folders):
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders["tinyA"])
    prompt = prompts_for(cfg, [3], seed=5)[0]
    want = P.greedy(cfg, w, prompt, 120)
    eng = engine(folders["tinyA"], kv_pool_tokens=256)
    assert eng.generate([prompt], SamplingParams(max_new_tokens=120)) == [want]


def test_stop_token_is_kept(folders):
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders["tinyA"])
    prompt = prompts_for(cfg, [12], seed=6)[0]
    free = P.greedy(cfg, w, prompt, 10)
    stop = free[4]
    cut = free[: free.index(stop) + 1]
    eng = engine(folders["tinyA"], kv_pool_tokens=256)
    assert eng.generate([prompt], SamplingParams(max_new_tokens=10, stop_token_ids=frozenset({stop}))) == [cut]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graph", [True, False])
def test_read_back_one_step_behind_changes_nothing(folders, dtype, graph):
    """The engine launches a step before it has read the previous one's tokens (they reach the next
    step on the device, through the uploaded ids or a captured graph's static buffer): same outputs
    as with a read-back after every step, with stop tokens that end requests one step late, sampled
    requests, and a pool that forces preemption."""
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders["tinyB"])
    prompts = prompts_for(cfg, [30, 45, 20, 38, 25, 41, 3, 17], seed=9)
    plain = {i: P.greedy(cfg, w, prompts[i], 6) for i in (2, 4)} if dtype == "float32" else {}  # greedy, no stops
    outs = {}
    for overlap in (True, False):
        eng = engine(folders["tinyB"], dtype, kv_pool_tokens=16 * 14, max_running=6, chunked_prefill_size=32,
                     decode_graph=graph, overlap=overlap)
        reqs = []
        for i, p in enumerate(prompts):
            stops = frozenset(range(0, cfg["vocab_size"], 9)) if i % 2 else frozenset()  # every ninth token ends odd requests
            reqs.append(eng.add_request(p, SamplingParams(20 + i, stop_token_ids=stops, temperature=0.0 if i % 3 else 0.9, seed=i)))
        while eng.has_unfinished:
            eng.step()
        assert eng.runner.cache.idle and all(r.in_flight == 0 for r in reqs)
        assert eng.scheduler.num_preemptions > 0, "the pool was meant to be too small"
        outs[overlap] = [r.output_ids for r in reqs]
        if overlap:
            assert eng.dropped_tokens > 0, "no request ran past a stop token"
            assert not graph or eng.runner.graph_steps > 0
    assert outs[True] == outs[False]
    for i, want in plain.items():
        assert outs[True][i][:6] == want


def test_a_step_returns_without_waiting_for_what_it_launches(folders):
    """With the read-back one step behind, ``step`` launches a batch and reads the tokens of the batch
    before it: it must not wait for the device to reach the new one. A long piece of device work is
    queued between two steps; the second step's own batch lies behind it, the batch it reads back ran
    before it, so the step returns long before that work ends. Without the overlap (the control: the
    measurement could not fail if this did not wait) the step reads its own batch back and takes as long
    as the queued work. Decode steps replayed from a graph and steps launched kernel by kernel alike."""
    import time

    import torch

    from miniserve_amd.engine.request import RequestState, SamplingParams

    cfg, _ = read_model_folder(folders["tinyB"])
    big = torch.randn((8192, 8192), device="cuda:0").to(torch.bfloat16)

    def busy():
        for _ in range(48):
            torch.matmul(big, big)

    busy()
    torch.cuda.synchronize()
    t = time.perf_counter()
    busy()
    torch.cuda.synchronize()
    busy_s = time.perf_counter() - t
    assert busy_s > 0.02, "the queued work is too short to measure against"
    for overlap, graph in ((True, True), (True, False), (False, True)):
        eng = engine(folders["tinyB"], "bfloat16", kv_pool_tokens=2048, max_running=4, decode_graph=graph, overlap=overlap)
        reqs = [eng.add_request(p, SamplingParams(max_new_tokens=60)) for p in prompts_for(cfg, [20, 33, 9, 41], seed=4)]
        while any(r.state is not RequestState.DECODE for r in reqs):
            eng.step()
        for _ in range(3):
            eng.step()
        torch.cuda.synchronize()
        eng.step()
        busy()
        t = time.perf_counter()
        eng.step()
        elapsed = time.perf_counter() - t
        torch.cuda.synchronize()
        if overlap:
            assert elapsed < 0.25 * busy_s, f"step took {elapsed * 1e3:.1f} ms with {busy_s * 1e3:.0f} ms of work queued ahead of its batch"
            assert not graph or eng.runner.graph_steps > 0
        else:
            assert elapsed > 0.8 * busy_s, f"the control did not wait: {elapsed * 1e3:.1f} ms of {busy_s * 1e3:.0f}"
        eng.overlap = not overlap  # switched between two steps: no token is lost or read twice
        while eng.has_unfinished:
            eng.step()
        assert eng.runner.cache.idle and all(len(r.output_ids) == 60 and r.in_flight == 0 for r in reqs)


def test_sampled_requests_reproduce_beside_greedy_ones(folders):
    """Temperature sampling with a request seed: the same tokens alone, in a batch, and after
    preemption; equal to the plain sampler run on the plain logits."""
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders["tinyB"])
    prompts = prompts_for(cfg, [14, 33, 21, 8], seed=7)
    params = [SamplingParams(12, temperature=t, top_p=tp, seed=s) for t, tp, s in
              ((0.8, 1.0, 11), (0.0, 1.0, None), (0.8, 0.9, 2**32 - 1), (1.5, 1.0, 0))]

    def plain_run(p, sp):
        ids, out = list(p), []
        for _ in range(sp.max_new_tokens):
            tok = P.sample(P.logits(cfg, w, ids)[-1], sp.temperature, sp.seed or 0, len(ids), sp.top_p)
            out.append(tok)
            ids.append(tok)
        return out

    want = [plain_run(p, sp) for p, sp in zip(prompts, params)]
    for pool in (1024, 16 * 7):
        eng = engine(folders["tinyB"], kv_pool_tokens=pool, max_running=4, chunked_prefill_size=16)
        reqs = [eng.add_request(p, sp) for p, sp in zip(prompts, params)]
        while eng.has_unfinished:
            eng.step()
        assert [r.output_ids for r in reqs] == want


def test_abort_gives_pages_back(folders):
    from miniserve_amd.engine.request import SamplingParams

    cfg, _ = read_model_folder(folders["tinyA"])
    eng = engine(folders["tinyA"], kv_pool_tokens=512, max_running=4)
    reqs = [eng.add_request(p, SamplingParams(50)) for p in prompts_for(cfg, [20, 30], seed=8)]
    for _ in range(5):
        eng.step()
    eng.abort(reqs[0].rid)
    eng.abort(reqs[0].rid)  # idempotent
    while eng.has_unfinished:
        eng.step()
    assert len(reqs[1].output_ids) == 50 and len(reqs[0].output_ids) < 50
    assert eng.runner.cache.idle


def test_bfloat16_generation_follows_its_logits_and_they_follow_plain(folders):
    """Greedy generation in bfloat16 through the entry point, with the logits of every sampling step
    taken from the engine's hook: they agree with the plain implementation's logits for the same prefix
    within the bfloat16 tolerance, every token is the first maximum of the engine's own logits, and it
    is the plain implementation's choice wherever that choice is clear of the tolerance (its lead over
    the runner-up is more than twice the largest error the tolerance allows)."""
    from miniserve_amd.engine.request import SamplingParams
    from tolerances import BF16_REL_MAX, check_logits

    for name in ("tinyB", "tinyD"):
        cfg, w = read_model_folder(folders[name])
        prompts = prompts_for(cfg, [25, 60], seed=9)
        eng = engine(folders[name], dtype="bfloat16", kv_pool_tokens=512, chunked_prefill_size=32)
        seen = {}  # rid -> list of logits rows, one per sampled token

        def hook(batch, logits):
            rows = [r for (r, _, _), done in zip(batch.rows, batch.completes()) if done]
            for r, row in zip(rows, logits.float().cpu().numpy()):
                seen.setdefault(r.rid, []).append(row)

        eng.logits_hook = hook
        reqs = [eng.add_request(p, SamplingParams(16)) for p in prompts]
        while eng.has_unfinished:
            eng.step()
        decisive = 0
        for p, r in zip(prompts, reqs):
            out = r.output_ids
            assert len(out) == 16 and len(seen[r.rid]) >= 16
            want = P.logits(cfg, w, p + out[:-1])[len(p) - 1 :]
            got = np.stack(seen[r.rid][:16])
            check_logits(got, want, "bfloat16", f"{name}: logits of the sampling steps")
            scale = float(np.abs(want).max())
            for i, tok in enumerate(out):
                assert tok == int(np.argmax(got[i])), "greedy takes the first maximum of the engine's logits"
                top = np.sort(want[i])[-2:]
                if top[1] - top[0] > 2 * BF16_REL_MAX * scale:
                    decisive += 1
                    assert tok == int(np.argmax(want[i])), f"{name}: token {i} differs from a clear choice of the plain implementation"
        assert decisive > 0, "no step had a clear choice: the comparison of tokens checked nothing"


def test_command_line_generate(folders):
    cfg, w = read_model_folder(folders["tinyA"])
    prompt = prompts_for(cfg, [6], seed=10)[0]
    res = subprocess.run(
        [sys.executable, "-m", "miniserve_amd", "generate", "--model", str(folders["tinyA"]), "--dtype", "float32",
         "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "8", "--kv-pool-tokens", "256"],
        capture_output=True, text=True, cwd=str(ROOT), timeout=110,
    )
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["outputs"] == [P.greedy(cfg, w, prompt, 8)]


def test_stress_run_finishes_and_returns_every_page(folders):
    res = subprocess.run(
        [sys.executable, "-m", "miniserve_amd", "stress", "--model", str(folders["tinyB"]), "--num-requests", "24",
         "--prompt-len", "4", "90", "--max-new-tokens", "1", "30", "--kv-pool-tokens", "640", "--max-running", "8",
         "--chunked-prefill-size", "64", "--temperature", "0.7", "--top-p", "0.9"],
        capture_output=True, text=True, cwd=str(ROOT), timeout=110,
    )
    assert res.returncode == 0, res.stdout[-1000:] + res.stderr[-2000:]
    report = json.loads(res.stdout.strip().splitlines()[-1])
    assert report["finished"] == 24 and report["idle"]
    # decode-only and mixed steps are timed apart; the effective configuration is read back from the engine
    assert report["decode_steps"]["steps"] > 0 and report["mixed_steps"]["steps"] > 0
    assert report["decode_steps"]["median_ms"] > 0 and report["mixed_steps"]["mean_tokens"] > report["decode_steps"]["mean_tokens"]
    eng = report["engine"]
    assert eng["kv_pool_tokens"] == [640] and eng["page_size"] == 16 and eng["chunked_prefill_size"] == 64
    assert eng["max_running"] == 8 and eng["architecture"] == "Qwen3ForCausalLM" and eng["overlap"] is True
    assert report["runtime"]["gpu"] and report["runtime"]["torch"]


def test_default_pool_is_sized_from_a_measured_peak(folders):
    """Without ``kv_pool_tokens`` the pool takes a share of what is free beyond the measured peak of
    the largest step (miniserve/engine/model_runner.py:152-203); the figures can be read back."""
    import torch

    from miniserve_amd.engine.describe import engine_description
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders["tinyD"])
    free, _ = torch.cuda.mem_get_info()
    eng = engine(folders["tinyD"], "bfloat16", max_running=4, chunked_prefill_size=256, kv_mem_fraction=0.02)
    prof = eng.runner.kv_profile
    assert prof["profile_tokens"] == 256 and prof["profile_sample_rows"] == 4
    assert prof["peak_activation_bytes"] > 256 * cfg["hidden_size"] * 4  # at least the float32 stream of the profiled step
    assert prof["decode_step_bytes"] > 0 and prof["graph_reserve_bytes"] == 4 * prof["decode_step_bytes"]
    assert prof["num_pages"] == prof["max_pages"] == int(0.02 * (prof["free_bytes"] - prof["peak_activation_bytes"]
                                                                 - prof["graph_reserve_bytes"])) // prof["bytes_per_page"]
    assert 0.01 * free < prof["pool_bytes"] <= 0.02 * prof["free_bytes"] + prof["bytes_per_page"]  # one page more: the dummy page
    d = engine_description(eng)
    assert d["kv_pool_pages"] == [prof["num_pages"]] and d["kv_profile"]["max_pages"] == prof["max_pages"]
    prompts = prompts_for(cfg, [30, 5])
    got = eng.generate(prompts, SamplingParams(max_new_tokens=6))
    assert [len(g) for g in got] == [6, 6] and eng.runner.cache.idle
    with pytest.raises(ValueError, match="fit in memory"):
        engine(folders["tinyD"], "bfloat16", kv_pool_tokens=2**40)


def test_a_windowed_group_gets_the_pages_it_can_use_and_the_rest_goes_to_the_others(folders):
    """tinyE keeps every key in two layers and a window of 100 in one. With prompts cut into portions of 64 a
    request never holds more than the window and a portion in the windowed layer: that group gets
    ``max_running * (pages(window - 1 + portion) + 1)`` pages, whether the pool is given in tokens or measured,
    and a measured pool spends what that saves on the other group. Generation is unchanged."""
    from miniserve_amd.engine.describe import engine_description
    from miniserve_amd.engine.request import SamplingParams

    cfg, w = read_model_folder(folders["tinyE"])
    need = 4 * (-(-(100 - 1 + 64) // 16) + 1)
    eng = engine(folders["tinyE"], "bfloat16", max_running=4, chunked_prefill_size=64, kv_pool_tokens=4096)
    assert [(g.window, n) for g, n in zip(eng.runner.layout.groups, eng.runner.cache.total_pages())] == [(0, 256), (100, need)]
    d = engine_description(eng)
    assert d["kv_pool_pages"] == [256, need] and d["kv_profile"]["pages_per_group"] == [256, need]
    prompts = prompts_for(cfg, [300, 40, 7])
    want = [P.greedy(cfg, w, p, 6) for p in prompts]
    ref = engine(folders["tinyE"], "float32", max_running=4, chunked_prefill_size=64, kv_pool_tokens=4096)
    assert ref.generate(prompts, SamplingParams(max_new_tokens=6)) == want and ref.runner.cache.idle
    del ref
    measured = engine(folders["tinyE"], "bfloat16", max_running=4, chunked_prefill_size=64, kv_mem_fraction=0.01)
    prof = measured.runner.kv_profile
    per_group = measured.runner.layout.bytes_per_page(16, 2)
    budget = int(0.01 * (prof["free_bytes"] - prof["peak_activation_bytes"] - prof["graph_reserve_bytes"]))
    assert prof["pages_per_group"] == [(budget - need * per_group[1]) // per_group[0], need]
    got = measured.generate(prompts, SamplingParams(max_new_tokens=6))
    assert [len(g) for g in got] == [6, 6, 6] and measured.runner.cache.idle
    # whole prompts run in one step however long: no bound on what the windowed group holds, it is sized like the other
    whole = engine(folders["tinyE"], "bfloat16", max_running=4, chunked_prefill_size=0, kv_pool_tokens=4096)
    assert whole.runner.cache.total_pages() == [256, 256]


def test_a_measured_pool_refuses_whole_prompts_beyond_the_step_it_was_measured_with(folders):
    """Whole prompts run in one step. A pool sized from the measured peak of a step of ``max_prefill_tokens`` tokens
    leaves no room for the activations of a longer step, so such a prompt is refused at submission; with a pool
    given in tokens nothing was measured and the prompt runs."""
    from miniserve_amd.engine.request import SamplingParams

    cfg, _ = read_model_folder(folders["tinyD"])
    long_prompt = prompts_for(cfg, [300])[0]
    eng = engine(folders["tinyD"], "bfloat16", max_running=2, chunked_prefill_size=0, max_prefill_tokens=128, kv_mem_fraction=0.01)
    assert eng.runner.kv_profile["profile_tokens"] == 128
    with pytest.raises(ValueError, match="use chunked prefill"):
        eng.add_request(long_prompt, SamplingParams(max_new_tokens=4))
    assert len(eng.generate([long_prompt[:100]], SamplingParams(max_new_tokens=4))[0]) == 4
    given = engine(folders["tinyD"], "bfloat16", max_running=2, chunked_prefill_size=0, max_prefill_tokens=128, kv_pool_tokens=1024)
    assert len(given.generate([long_prompt], SamplingParams(max_new_tokens=4))[0]) == 4
