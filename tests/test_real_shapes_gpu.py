"""The benchmark's layer sizes (Qwen3-0.6B: hidden 1024, 16/8 heads of 128, intermediate 3072, vocabulary
151,936) with two layers and random weights: the float32 path against the plain implementation, its
bitwise independence of how the prompt is cut, and bfloat16 against float32."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P
from plain.model_folder import read_model_folder
from tolerances import check_logits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from miniserve_amd.config.presets import preset
    from miniserve_amd.weights.random_init import Init, write_model_folder

    cfg = preset("0.6B")
    cfg["num_hidden_layers"] = 2
    return write_model_folder(tmp_path_factory.mktemp("real") / "m", cfg, 5, Init(0.02, (0.8, 1.2)))


def run(folder, dtype, ids, cuts, want_last):
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import load_model

    runner = ModelRunner(load_model(folder, dtype), kv_pool_tokens=1024, max_running=2)
    rc = runner.acquire()
    out, at = [], 0
    for n in cuts:
        wanted = [i for i in range(n) if at + i >= len(ids) - want_last]
        logits = runner.step([StepRow(rc, ids[at : at + n], wanted)])
        if wanted:
            out.append(logits.cpu())
        at += n
    runner.release(rc)
    return torch.cat(out)


def test_benchmark_shapes(folder):
    rng = np.random.default_rng(1)
    T, last = 300, 40
    ids = rng.integers(0, 150000, T).tolist()
    whole = run(folder, "float32", ids, [T], last)
    cut = run(folder, "float32", ids, [130, 70, 60] + [1] * 40, last)
    assert torch.equal(whole, cut), "float32 logits must not depend on how the prompt is cut"
    cfg, w = read_model_folder(folder)
    h = P.hidden_states(cfg, w, ids)
    c = P.read_config(cfg)
    want = P.rms_norm(h[-last:], w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T
    check_logits(whole.numpy(), want, "float32", "0.6B shape float32 whole")
    for cuts in ([T], [130, 70, 60] + [1] * 40):
        check_logits(run(folder, "bfloat16", ids, cuts, last).numpy(), want, "bfloat16", f"0.6B shape bfloat16 {cuts[:3]}")
