"""Configurations drawn at random (head sizes 16..256 in steps of 16, any number of heads and groups,
widths and vocabularies that are no power of two and no multiple of 8, windows on some layers given
by either set of config.json keys), each replayed as a mixed trace with page reuse through the step
function and compared with the plain implementation in float32 and in bfloat16."""

from __future__ import annotations

import numpy as np
import pytest

from miniserve_amd.weights.random_init import Init, write_model_folder
from plain import qwen3_plain as P
from plain.model_folder import read_model_folder
from test_replay_gpu import mixed_schedule
from tolerances import check_logits

pytestmark = pytest.mark.gpu


def draw_config(rng, medium: bool) -> dict:
    if medium:  # sizes at which rows of 17 and more take the matrix-core tile kernels
        D = int(rng.choice([64, 128]))
        Hkv, G = int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4, 6, 8, 16]))
        L = int(rng.integers(1, 4))
        hidden = int(rng.choice([256, 384, 512, 576, 1024, 328]))
        inter = int(rng.choice([512, 768, 1000, 1536, 1088]))
        vocab = int(rng.integers(1000, 6000))
    else:
        D = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 192, 256]))
        Hkv, G = int(rng.choice([1, 2, 3, 4, 5])), int(rng.choice([1, 1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 20]))
        if D >= 144:
            G, Hkv = min(G, 4), min(Hkv, 2)
        L = int(rng.integers(1, 5))
        hidden = int(rng.choice([24, 40, 56, 64, 72, 88, 100, 130, 200, 250, 67, 96, 128, 264, 320]))
        inter = int(rng.choice([40, 56, 100, 136, 176, 224, 250, 333, 512, 48, 1000]))
        vocab = int(rng.integers(50, 1500))
    cfg = dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=L,
        hidden_size=hidden, num_attention_heads=Hkv * G, num_key_value_heads=Hkv, head_dim=D,
        intermediate_size=inter, vocab_size=vocab, rope_theta=float(rng.choice([1e4, 5e4, 1e6])),
        rms_norm_eps=float(rng.choice([1e-6, 1e-5, 3e-6])), tie_word_embeddings=bool(rng.random() < 0.5),
        max_position_embeddings=4096,
    )
    mode = int(rng.integers(0, 3))
    if mode == 1:
        cfg["sliding_window"] = int(rng.choice([1, 2, 5, 16, 17, 31, 32, 33, 64, 70]))
        cfg["layer_types"] = [str(rng.choice(["sliding_attention", "full_attention"])) for _ in range(L)]
    elif mode == 2:
        cfg["sliding_window"] = int(rng.choice([3, 8, 16, 24, 48, 100]))
        cfg["use_sliding_window"] = True
        cfg["max_window_layers"] = int(rng.integers(0, L + 1))
    return cfg


@pytest.mark.parametrize("medium", (False, True), ids=("small", "medium"))
@pytest.mark.parametrize("seed", range(6))
def test_random_configuration(seed, medium, tmp_path):
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import load_model

    rng = np.random.default_rng(1000 * medium + seed)
    cfg = draw_config(rng, medium)
    folder = write_model_folder(tmp_path / "m", cfg, seed, Init(float(rng.choice([0.02, 0.05, 0.08])), (0.5, 1.5)))
    pcfg, w = read_model_folder(folder)
    pool = [1, 2, 3, 9, 17, 31, 33, 64, 65, 100, 127, 129, 200, 260] + ([300, 513] if medium else [])
    lengths = [int(x) for x in rng.choice(pool, size=int(rng.integers(3, 6)))]
    reqs = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in lengths]
    want = [P.logits(pcfg, w, ids) for ids in reqs]
    steps, peak = mixed_schedule(lengths, seed=seed)
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner(load_model(folder, dtype, "cuda:0"), page_size=16, kv_pool_tokens=peak, max_running=8)
        live = {}
        for entries, ends in steps:
            rows = []
            for i, s, n in entries:
                if i not in live:
                    live[i] = runner.acquire()
                rows.append(StepRow(live[i], reqs[i][s : s + n], list(range(n))))
            got = runner.step(rows).float().cpu().numpy()
            at = 0
            for i, s, n in entries:
                check_logits(got[at : at + n], want[i][s : s + n], dtype, f"{cfg} request {i} tokens {s}..{s + n}")
                at += n
            for i in ends:
                runner.release(live.pop(i))
        assert runner.cache.idle, "pages were not all given back"


@pytest.mark.parametrize("name", ("tinyD", "tinyE"))
def test_portions_with_keys_in_parts(name, tmp_path, monkeypatch):
    """Portions of prompts beside single tokens with the prefill attention forced to hand the keys of
    every tile deeper than four key tiles out in parts (the host's own rule does so only far into long
    sequences): the step function's logits still follow the plain implementation. tinyD has head
    size 64, tinyE head size 128 and a windowed layer, which keeps whole tiles."""
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.kernels import ops
    from miniserve_amd.loading import load_model
    from models import make_folder

    monkeypatch.setattr(ops, "PREFILL_PARTS_LAUNCH_US", -1e9)
    folder = make_folder(tmp_path, name)
    pcfg, w = read_model_folder(folder)
    rng = np.random.default_rng(5)
    lengths = [700, 330, 90]
    reqs = [rng.integers(0, pcfg["vocab_size"], size=n).tolist() for n in lengths]
    want = [P.logits(pcfg, w, ids) for ids in reqs]
    runner = ModelRunner(load_model(folder, "bfloat16", "cuda:0"), page_size=16, kv_pool_tokens=1280, max_running=4)
    rcs = [runner.acquire() for _ in reqs]
    fed = [0, 0, 0]
    taken = 0
    for portion in (300, 64, 200, 33, 128, 2, 400):
        rows, spans = [], []
        for i, n in enumerate(lengths):
            k = min(portion if i != 2 else 1, n - fed[i])  # the third request goes one token at a time
            if k > 0:
                rows.append(StepRow(rcs[i], reqs[i][fed[i] : fed[i] + k], list(range(k))))
                spans.append((i, fed[i], k))
                fed[i] += k
        if not rows:
            break
        plan = ops.plan_prefill_parts([k for _, _, k in spans], [s for _, s, _ in spans], 32, 1)
        taken += plan is not None
        got = runner.step(rows).float().cpu().numpy()
        at = 0
        for i, s, k in spans:
            check_logits(got[at : at + k], want[i][s : s + k], "bfloat16", f"{name} request {i} tokens {s}..{s + k}")
            at += k
    assert taken >= 3, "the steps were meant to have tiles deep enough to be cut"
    for rc in rcs:
        runner.release(rc)
    assert runner.cache.idle
