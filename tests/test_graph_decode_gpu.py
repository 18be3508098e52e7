"""The path the benchmark times, against the plain implementation: bfloat16 decode steps replayed from
captured graphs, with the matrix-core decode attention (head sizes 64 and 128, 16-token pages), rows
of padding on the dummy page (3 and 5 live rows in buckets of 4 and 8), sequences that grow across a
table-width bucket (256 -> 257 tokens: 16 -> 32 table entries), a request released under way and its
pages taken by a new one, and a windowed layer (tinyE) whose tables hold entries that were given
back. Every logit of every step is compared, teacher-forced."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from models import make_folder
from plain import qwen3_plain as P
from plain.model_folder import read_model_folder
from tolerances import check_logits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from miniserve_amd.config.presets import preset
    from miniserve_amd.weights.random_init import Init, write_model_folder

    root = tmp_path_factory.mktemp("graphs")
    big = preset("0.6B")
    big["num_hidden_layers"] = 2
    return {"tinyD": make_folder(root, "tinyD"), "tinyE": make_folder(root, "tinyE"),
            "0.6B-2": write_model_folder(root / "big", big, 7, Init(0.02, (0.8, 1.2)))}


class Plain:
    """Logits of whole sequences, head applied only where asked (the large vocabulary)."""

    def __init__(self, folder):
        self.cfg, self.w = read_model_folder(folder)
        self.c = P.read_config(self.cfg)
        self.hidden = {}

    def rows(self, key, ids, places):
        if key not in self.hidden:
            self.hidden[key] = P.hidden_states(self.cfg, self.w, ids)
        h = self.hidden[key][places]
        return P.rms_norm(h, self.w["model.norm.weight"], self.c["eps"]) @ self.w["lm_head.weight"].T


@pytest.mark.parametrize("name", ["tinyD", "tinyE", "0.6B-2"])
def test_graph_replayed_decode_against_plain(name, folders):
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import load_model

    plain = Plain(folders[name])
    vocab = min(plain.cfg["vocab_size"], 150000)
    rng = np.random.default_rng(11)
    decode = 24
    lens = {"a": 250, "b": 3, "c": 100, "d": 255, "e": 17, "f": 40}
    seqs = {k: rng.integers(0, vocab, n + decode).tolist() for k, n in lens.items()}
    pages = sum(-(-(n + decode) // 16) for k, n in lens.items() if k != "f") + 1
    runner = ModelRunner(load_model(folders[name], "bfloat16"), kv_pool_tokens=16 * pages, max_running=8,
                         decode_graph=True, decode_graph_max_bs=8)
    assert runner.graphs is not None
    cache = {k: runner.acquire() for k in "abcde"}
    fed = dict.fromkeys(lens, 0)
    checked = 0

    def step(entries):
        """entries: (key, number of tokens); the last position of every row is compared."""
        nonlocal checked
        rows = [StepRow(cache[k], seqs[k][fed[k] : fed[k] + n], [n - 1]) for k, n in entries]
        got = runner.step(rows).float().cpu().numpy()
        for i, (k, n) in enumerate(entries):
            fed[k] += n
            want = plain.rows(k, seqs[k], [fed[k] - 1])
            check_logits(got[i : i + 1], want, "bfloat16", f"{name} request {k} position {fed[k] - 1}")
            checked += 1

    step([(k, lens[k]) for k in "abcde"])  # the prompts, one step, no graph
    graphs_before = runner.graph_steps
    live = list("abcde")
    for i in range(decode - 1):
        if i == 8:
            left = [set(t.pages) - {-1} for t in cache["c"].tables]
            runner.release(cache.pop("c"))  # its pages are the next to be handed out
            live.remove("c")
        if i == 10:
            cache["f"] = runner.acquire()
            step([(k, 1) for k in live] + [("f", lens["f"])])  # a mixed step: eager
            for g, t, was_c in zip(runner.layout.groups, cache["f"].tables, left):
                if not g.window:  # (a windowed group's newest free pages are those the other requests' windows just passed)
                    assert set(t.pages) <= was_c, "the new request was meant to run in the pages the released one held"
            live.append("f")
            continue
        if i == 16:
            for k in ("a", "e"):
                runner.release(cache.pop(k))
                live.remove(k)
        step([(k, 1) for k in live])
    assert runner.graph_steps - graphs_before == decode - 2, "every step of single tokens replays a graph"
    keys = set(runner.graphs.captured)
    assert {g for g, _ in keys} == {4, 8}, keys  # 5 and 4 rows in the bucket of 8 and 4, then 3 rows in the bucket of 4
    assert {w for _, w in keys} == {16, 32}, keys  # a and d grow past 256 tokens
    assert checked == 5 + 8 * 5 + 2 * 4 + 5 + 5 * 5 + 7 * 3
    for k in list(cache):
        runner.release(cache.pop(k))
    assert runner.cache.idle
