"""The benchmark shapes' layer sizes with random weights, as models against the plain implementation:
Qwen3-0.6B (hidden 1024, 16/8 heads of 128, intermediate 3072, tied head; two layers), Qwen3-8B
(hidden 4096, 32/8 heads, intermediate 12288; one layer) and Qwen3-32B (hidden 5120, 64/8 heads,
intermediate 25600; one layer), each with the full vocabulary of 151,936. Per shape: the float32 path
is bitwise independent of how the prompt is cut and of what else is in the batch (a portion beside
single tokens of another request), float32 and bfloat16 agree with the plain implementation.

The weights are drawn once on the GPU and handed to both the engine and the plain implementation
(no folder: the large shapes are several GB)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P
from tolerances import check_logits

pytestmark = pytest.mark.gpu

SHAPES = {"0.6B": 2, "8B": 1, "32B": 1}  # preset -> layers


@pytest.fixture(scope="module", params=sorted(SHAPES))
def shape(request):
    from miniserve_amd.config.presets import preset
    from miniserve_amd.config.registry import config_from_dict
    from miniserve_amd.weights.random_init import Init, random_tensors

    cfg = preset(request.param)
    cfg["num_hidden_layers"] = SHAPES[request.param]
    spec = config_from_dict(cfg).to_spec()
    tensors = random_tensors(spec, 5, Init(0.02, (0.8, 1.2)), dtype=torch.bfloat16, device="cuda:0")
    w = {k: v.float().cpu().numpy().astype(np.float64) for k, v in tensors.items()}
    if cfg.get("tie_word_embeddings"):
        w["lm_head.weight"] = w["model.embed_tokens.weight"]
    yield request.param, cfg, spec, tensors, w
    del tensors
    torch.cuda.empty_cache()


def model(spec, tensors, dtype):
    from miniserve_amd.loading import runtime
    from miniserve_amd.parts.model import DecoderModel

    rt = runtime(dtype)
    return DecoderModel(spec, {k: v.to(rt.dtype) for k, v in tensors.items()}, rt)


def run(m, ids, cuts, want_last, beside=None):
    """Feed ``ids`` in portions of ``cuts`` and return the logits of the last ``want_last`` positions.
    ``beside = (ids2, step)``: a second request whose prompt but for the last token runs beside the
    first portion and whose last token runs, as a single token, beside portion ``step``; its logits
    are returned too."""
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner

    runner = ModelRunner(m, kv_pool_tokens=1024, max_running=2)
    rc = runner.acquire()
    other = runner.acquire() if beside else None
    out, at, extra = [], 0, None
    for i, n in enumerate(cuts):
        wanted = [j for j in range(n) if at + j >= len(ids) - want_last]
        rows = [StepRow(rc, ids[at : at + n], wanted)]
        if beside and i == 0:
            rows.append(StepRow(other, beside[0][:-1], []))
        if beside and i == beside[1]:
            rows.insert(0, StepRow(other, beside[0][-1:], [0]))
        logits = runner.step(rows)
        if beside and i == beside[1]:
            extra, logits = logits[:1].cpu(), logits[1:]
        if wanted:
            out.append(logits.cpu())
        at += n
    runner.release(rc)
    if other is not None:
        runner.release(other)
    assert runner.cache.idle
    return (torch.cat(out), extra) if beside else torch.cat(out)


def test_layer_sizes_of_the_benchmark_shapes(shape):
    name, cfg, spec, tensors, w = shape
    rng = np.random.default_rng(1)
    T, last = 300, 40
    ids = rng.integers(0, 150000, T).tolist()
    ids2 = rng.integers(0, 150000, 80).tolist()
    c = P.read_config(cfg)

    def plain_rows(seq, places):
        h = P.hidden_states(cfg, w, seq)[places]
        return P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T

    want = plain_rows(ids, slice(T - last, T))
    want2 = plain_rows(ids2, slice(79, 80))
    cuts = [130, 70, 60] + [1] * 40
    m = model(spec, tensors, "float32")
    whole = run(m, ids, [T], last)
    cut = run(m, ids, cuts, last)
    assert torch.equal(whole, cut), f"{name}: float32 logits must not depend on how the prompt is cut"
    mixed, single = run(m, ids, [200, 60, 40], last, beside=(ids2, 1))
    assert torch.equal(whole, mixed), f"{name}: float32 logits must not depend on what else is in the batch"
    check_logits(whole.numpy(), want, "float32", f"{name} shape float32 whole")
    check_logits(single.numpy(), want2, "float32", f"{name} shape float32, a single token beside a portion")
    del m
    torch.cuda.empty_cache()
    m = model(spec, tensors, "bfloat16")
    for how in ([T], cuts):
        check_logits(run(m, ids, how, last).numpy(), want, "bfloat16", f"{name} shape bfloat16 {how[:3]}")
    mixed, single = run(m, ids, [200, 60, 40], last, beside=(ids2, 1))
    check_logits(mixed.numpy(), want, "bfloat16", f"{name} shape bfloat16 mixed")
    check_logits(single.numpy(), want2, "bfloat16", f"{name} shape bfloat16, a single token beside a portion")


def test_a_2048_token_step_of_the_32B_layer(shape, monkeypatch):
    """One step of 2,048 prompt tokens at the 32B layer sizes, bfloat16: eight query heads per KV head make
    16-token attention blocks, 1,024 of them, so this step (and every step of that shape's benchmark) runs
    the prefill attention's 128-row blocks and the matrix products' largest tiles. The last 40 positions'
    logits against the plain implementation."""
    name, cfg, spec, tensors, w = shape
    if name != "32B":
        pytest.skip("only the 32B shape's group of eight heads reaches the 128-row blocks at 2,048 tokens")
    from miniserve_amd.kernels import ops

    lib, seen = ops.library(), []
    for fn, at in (("ms_attention_prefill_bf16", 9), ("ms_attention_prefill_parts_bf16", 11)):
        real = getattr(lib, fn)
        monkeypatch.setattr(lib, fn, lambda *a, _real=real, _at=at: (seen.append(a[_at]), _real(*a))[1])
    rng = np.random.default_rng(2)
    T, last = 2048, 40
    ids = rng.integers(0, 150000, T).tolist()
    c = P.read_config(cfg)
    h = P.hidden_states(cfg, w, ids)[T - last :]
    want = P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T
    m = model(spec, tensors, "bfloat16")
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner

    runner = ModelRunner(m, kv_pool_tokens=4096, max_running=2)
    rc = runner.acquire()
    got = runner.step([StepRow(rc, ids, list(range(T - last, T)))]).float().cpu().numpy()
    assert seen and set(seen) == {128}, seen
    check_logits(got, want, "bfloat16", "32B shape bfloat16, 2,048 tokens in one step")
    # and the next portion behind it, beside nothing: 600 more tokens whose blocks (38 x 8) are few again
    more = rng.integers(0, 150000, 600).tolist()
    h = P.hidden_states(cfg, w, ids + more)[-last:]
    want = P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T
    got = runner.step([StepRow(rc, more, list(range(600 - last, 600)))]).float().cpu().numpy()
    assert seen[-1] == 64, seen
    check_logits(got, want, "bfloat16", "32B shape bfloat16, 600 tokens behind 2,048")
    runner.release(rc)
