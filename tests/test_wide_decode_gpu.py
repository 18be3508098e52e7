"""Decode steps of 17, 33 and 64 rows as whole models against the plain implementation, in bfloat16,
replayed from captured graphs. Above 16 rows a step takes other kernels than the small batches the
other tests run: the reduction of the key splits on its own (no merged output projection), the
activation kernel on partial sums, products as 64 x 64 tiles with K split, and at 64 rows one key
split. Every row's logits at every step are compared, teacher-forced; the sequences differ in
length (some shorter than a page, some several hundred tokens, one that crosses a table-width bucket).
The weights are random: what this pins is the composition of the kernels, which each have a test of
their own with inputs made so that a skipped key shows."""

from __future__ import annotations

import numpy as np
import pytest

from models import make_folder
from plain import qwen3_plain as P
from plain.model_folder import read_model_folder
from tolerances import check_logits

pytestmark = pytest.mark.gpu

DECODE = 4


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from miniserve_amd.config.presets import preset
    from miniserve_amd.weights.random_init import Init, write_model_folder

    root = tmp_path_factory.mktemp("wide")
    big = preset("0.6B")
    big["num_hidden_layers"] = 2
    return {"tinyD": make_folder(root, "tinyD"), "tinyE": make_folder(root, "tinyE"),
            "0.6B-2": write_model_folder(root / "big", big, 9, Init(0.02, (0.8, 1.2)))}


def plain_rows(cfg, w, c, ids, places):
    h = P.hidden_states(cfg, w, ids)[places]
    return P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T


@pytest.mark.parametrize("rows", [17, 33, 64])
@pytest.mark.parametrize("name", ["tinyD", "tinyE", "0.6B-2"])
def test_wide_decode_steps_against_plain(name, rows, folders):
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import load_model

    cfg, w = read_model_folder(folders[name])
    c = P.read_config(cfg)
    vocab = min(cfg["vocab_size"], 150000)
    rng = np.random.default_rng(rows)
    # lengths: page edges, one token, a few hundred; row 0 crosses 256 tokens (a wider table bucket) while decoding
    lens = [254, 1, 15, 16, 17, 300, 600][: min(rows, 7)] + rng.integers(2, 200, max(0, rows - 7)).tolist()
    seqs = [rng.integers(0, vocab, n + DECODE).tolist() for n in lens]
    pages = sum(-(-(n + DECODE) // 16) for n in lens) + 2
    runner = ModelRunner(load_model(folders[name], "bfloat16"), kv_pool_tokens=16 * pages, max_running=rows,
                         decode_graph=True, decode_graph_max_bs=rows)
    caches = [runner.acquire() for _ in lens]
    # prompts in steps of at most 16 rows (what the prompt path is tested with elsewhere)
    for a in range(0, rows, 16):
        runner.step([StepRow(caches[i], seqs[i][: lens[i]], []) for i in range(a, min(rows, a + 16))])
    want = [plain_rows(cfg, w, c, s, slice(n, n + DECODE)) for s, n in zip(seqs, lens)]
    before = runner.graph_steps
    for j in range(DECODE):
        got = runner.step([StepRow(caches[i], [seqs[i][lens[i] + j]], [0]) for i in range(rows)]).float().cpu().numpy()
        for i in range(rows):
            check_logits(got[i : i + 1], want[i][j : j + 1], "bfloat16", f"{name}: {rows} rows, row {i} (length {lens[i] + j + 1})")
    assert runner.graph_steps - before == DECODE, "every step of single tokens replays a graph"
    assert {g for g, _ in runner.graphs.captured} == {rows}
    for rc in caches:
        runner.release(rc)
    assert runner.cache.idle
