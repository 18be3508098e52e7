"""Pins of the plain implementation beside the reference's text: special cases that reduce to a
library routine, and invariants, each chosen so that a plausible mistake fails it (a wrong sign or
pairing in the rotation, a norm in the wrong place or with the wrong eps, a mask off by one, a wrong
head-to-group map), and for the wiring of a layer (which norm feeds what, the per-head norms before the
rotation, q_norm against k_norm, pre-norm residual sums, the final norm) a one-layer special case worked
out in complex arithmetic plus what zeroed weights must switch off. The reference's own numeric tests
compare with a library model on downloaded weights (tests/test_consistency.py:68-145) and hold no
vectors that could be reused here."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from models import TINY
from miniserve_amd.weights.random_init import write_model_folder
from plain import qwen3_plain as P
from plain.model_folder import read_model_folder

rng = np.random.default_rng(0)


# ------------------------------------------------------------------------------------------ norm


def test_rms_norm_formula_and_eps():
    x = rng.standard_normal((5, 12)) * 3
    w = rng.uniform(0.5, 1.5, 12)
    eps = 1e-5
    want = x / np.sqrt((x**2).mean(-1, keepdims=True) + eps) * w
    assert np.allclose(P.rms_norm(x, w, eps), want, rtol=1e-14)
    ones = np.ones(12)
    y = P.rms_norm(x, ones, eps)
    ms = (x**2).mean(-1)
    assert np.allclose((y**2).mean(-1), ms / (ms + eps), rtol=1e-12)  # the weight is plain, not 1 + w
    assert np.allclose(P.rms_norm(7 * x, ones, 0.0), P.rms_norm(x, ones, 0.0), rtol=1e-12)  # scale-free as eps -> 0
    small = x * 1e-3
    assert np.abs(P.rms_norm(small, ones, 1e-6) - P.rms_norm(small, ones, 1e-5)).max() > 1e-2  # eps really enters
    assert not np.allclose(P.rms_norm(x, w, eps), x - x.mean(-1, keepdims=True))  # no mean is removed


# ------------------------------------------------------------------------------------------ rotation


def test_rotary_frequencies():
    ang = P.rotary_angles(np.array([0, 1, 5]), 8, 10000.0)
    assert ang.dtype == np.float32 and ang.shape == (3, 4)
    assert np.all(ang[0] == 0) and ang[1, 0] == 1.0
    assert np.allclose(ang[1], 10000.0 ** (-np.arange(0, 8, 2) / 8), rtol=1e-6)
    assert np.allclose(ang[2], 5 * ang[1], rtol=1e-6)


def test_rotation_pairs_j_with_j_plus_half_and_turns_counterclockwise():
    d = 8
    ang = P.rotary_angles(np.array([3]), d, 100.0)
    x = np.zeros((1, 1, d))
    x[0, 0, 1] = 1.0  # the first element of pair (1, 1 + d/2)
    y = P.apply_rotary(x, ang)[0, 0]
    a = float(ang[0, 1])
    want = np.zeros(d)
    want[1], want[1 + d // 2] = np.cos(a), np.sin(a)
    assert np.allclose(y, want, atol=1e-12)  # interleaved pairing would put the sine at index 0 or 2
    x = np.zeros((1, 1, d))
    x[0, 0, 1 + d // 2] = 1.0
    y = P.apply_rotary(x, ang)[0, 0]
    want = np.zeros(d)
    want[1], want[1 + d // 2] = -np.sin(a), np.cos(a)
    assert np.allclose(y, want, atol=1e-12)


def test_rotation_invariants():
    d = 16
    q, k = rng.standard_normal((1, 1, d)), rng.standard_normal((1, 1, d))
    at = lambda x, p: P.apply_rotary(x, P.rotary_angles(np.array([p]), d, 10000.0))[0, 0]
    assert np.allclose(at(q, 0), q[0, 0])  # position 0 is the identity
    r = at(q, 7)
    assert np.allclose(r[: d // 2] ** 2 + r[d // 2 :] ** 2, q[0, 0, : d // 2] ** 2 + q[0, 0, d // 2 :] ** 2)  # pair norms
    dots = [at(q, m) @ at(k, n) for m, n in ((5, 2), (13, 10), (103, 100))]
    assert np.allclose(dots, dots[0], rtol=1e-5)  # only the distance counts
    assert abs(at(q, 5) @ at(k, 2) - at(q, 2) @ at(k, 5)) > 1e-3  # and its sign


# ------------------------------------------------------------------------------------------ attention


def sdpa(q, k, v, scale, causal):
    t = lambda x: torch.from_numpy(x).permute(1, 0, 2)[None]
    out = F.scaled_dot_product_attention(t(q), t(k), t(v), is_causal=causal, scale=scale, enable_gqa=True)
    return out[0].permute(1, 0, 2).numpy()


@pytest.mark.parametrize("hq,hkv", [(4, 4), (6, 2), (6, 1), (1, 1)])
def test_attention_reduces_to_the_library_routine(hq, hkv):
    T, d = 9, 8
    q, k, v = rng.standard_normal((T, hq, d)), rng.standard_normal((T, hkv, d)), rng.standard_normal((T, hkv, d))
    assert np.allclose(P.attention(q, k, v, 0.3), sdpa(q, k, v, 0.3, True), atol=1e-12)
    # the last query sees every key: no mask at all
    assert np.allclose(P.attention(q, k, v, 0.3)[-1:], sdpa(q[-1:], k, v, 0.3, False), atol=1e-12)


def test_attention_special_cases():
    d = 8
    q, k, v = rng.standard_normal((1, 2, d)), rng.standard_normal((1, 1, d)), rng.standard_normal((1, 1, d))
    assert np.allclose(P.attention(q, k, v, 1.0)[0], np.broadcast_to(v[0], (2, d)))  # one token: o = v
    T = 6
    q = rng.standard_normal((T, 1, d))
    k = np.broadcast_to(rng.standard_normal((1, 1, d)), (T, 1, d)).copy()
    v = rng.standard_normal((T, 1, d))
    out = P.attention(q, k, v, 0.7)
    for t in range(T):
        assert np.allclose(out[t, 0], v[: t + 1, 0].mean(0))  # equal keys: the mean of the values seen
    # head h reads KV head h // group
    hq, hkv = 6, 3
    q = rng.standard_normal((1, hq, d))
    k = rng.standard_normal((1, hkv, d))
    v = np.arange(hkv, dtype=float)[None, :, None] * np.ones((1, hkv, d))
    assert np.allclose(P.attention(q, k, v, 1.0)[0, :, 0], [0, 0, 1, 1, 2, 2])


def test_window_meaning():
    T, d = 12, 8
    q, k, v = rng.standard_normal((T, 2, d)), rng.standard_normal((T, 1, d)), rng.standard_normal((T, 1, d))
    assert np.allclose(P.attention(q, k, v, 0.5, window=T), P.attention(q, k, v, 0.5))
    assert np.allclose(P.attention(q, k, v, 0.5, window=1), np.broadcast_to(v, (T, 2, d)))  # only itself
    w3 = P.attention(q, k, v, 0.5, window=3)
    for t in (2, 7, 11):  # the last three keys, as a short sequence of its own
        lo = max(0, t - 2)
        assert np.allclose(w3[t], P.attention(q[lo : t + 1], k[lo : t + 1], v[lo : t + 1], 0.5)[-1])


def test_swiglu():
    x = rng.standard_normal((4, 6))
    wg, wu, wd = rng.standard_normal((10, 6)), rng.standard_normal((10, 6)), rng.standard_normal((6, 10))
    g = x @ wg.T
    assert np.allclose(P.swiglu(x, wg, wu, wd), (g / (1 + np.exp(-g)) * (x @ wu.T)) @ wd.T)
    assert P.silu(np.zeros(3)).tolist() == [0, 0, 0] and np.isclose(P.silu(np.array([20.0]))[0], 20.0)
    assert not np.allclose(P.swiglu(x, wg, wu, wd), P.swiglu(x, wu, wg, wd))  # gate and up are not interchangeable


def test_the_reference_says_both_formulas_twice():
    """The direction of the turn and which of gate / up goes through SiLU are stated twice in the reference, in
    different words: once as written-out arithmetic (model/qwen3.py:85-87,107-108,128-131, what ``tests/plain``
    follows) and once as calls of library operators in its fused path, whose published meanings are fixed
    outside the reference: ``apply_rope_with_cos_sin_cache_inplace(..., is_neox=True)`` over a table of one
    row ``[cos(angles), sin(angles)]`` per token (model/fused.py:182-184,209: the halves of a head are the
    pairs, ``first' = first cos - second sin``, ``second' = second cos + first sin``), and ``silu_and_mul``
    over the product with the concatenated weight, gate rows first (model/fused.py:41,195:
    ``silu(y[..., :I]) * y[..., I:]``). The reference's own tests hold the two paths equal on a real checkpoint
    (tests/test_fused.py:71-141). Written here from the second statement and compared with the first."""
    d, t = 16, 5
    x = rng.standard_normal((t, 3, d))
    pos = np.array([0, 1, 7, 300, 4000])
    ang = P.rotary_angles(pos, d, 1e6).astype(np.float64)
    table = np.concatenate((np.cos(ang), np.sin(ang)), axis=-1)  # one row per token: cosines, then sines
    cos, sin = table[:, None, : d // 2], table[:, None, d // 2 :]
    first, second = x[..., : d // 2], x[..., d // 2 :]
    neox = np.concatenate((first * cos - second * sin, second * cos + first * sin), axis=-1)
    assert np.allclose(P.apply_rotary(x, ang.astype(np.float32)), neox, atol=1e-12)
    other_way = np.concatenate((first * cos + second * sin, second * cos - first * sin), axis=-1)
    assert not np.allclose(neox, other_way)
    h, inter = 6, 10
    y = rng.standard_normal((4, h))
    wg, wu, wd = rng.standard_normal((inter, h)), rng.standard_normal((inter, h)), rng.standard_normal((h, inter))
    both = y @ np.concatenate((wg, wu), axis=0).T  # gate rows first
    silu_and_mul = both[:, :inter] / (1 + np.exp(-both[:, :inter])) * both[:, inter:]
    assert np.allclose(P.swiglu(y, wg, wu, wd), silu_and_mul @ wd.T)


# ------------------------------------------------------------------------------------------ the whole model


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("plain")
    return {n: read_model_folder(write_model_folder(root / n, cfg, seed, init)) for n, (cfg, seed, init) in TINY.items()}


@pytest.mark.parametrize("name", sorted(TINY))
def test_only_distances_between_positions_count(name, models):
    cfg, w = models[name]
    ids = rng.integers(0, cfg["vocab_size"], 20)
    base = P.logits(cfg, w, ids)
    shifted = P.logits(cfg, w, ids, positions=np.arange(20) + 37)
    assert np.abs(shifted - base).max() < 2e-4 * np.abs(base).max()  # float32 angles: equal up to their rounding
    later = np.arange(20)
    later[10:] += 1  # a gap in the middle is not a shift of all positions
    assert np.abs(P.logits(cfg, w, ids, positions=later)[10:] - base[10:]).max() > 1e-3 * np.abs(base).max()


@pytest.mark.parametrize("name", sorted(TINY))
def test_causality_and_dependence(name, models):
    cfg, w = models[name]
    ids = rng.integers(0, cfg["vocab_size"], 40)
    base = P.logits(cfg, w, ids)
    other = ids.copy()
    other[25] = (other[25] + 1) % cfg["vocab_size"]
    changed = P.logits(cfg, w, other)
    assert np.array_equal(changed[:25], base[:25])  # a token never changes what came before it
    assert np.abs(changed[25:] - base[25:]).max() > 1e-6
    assert np.allclose(P.logits(cfg, w, ids[:17]), base[:17], rtol=0, atol=1e-12)  # a prefix is a prefix


def test_window_layers_forget_far_tokens(models):
    cfg, w = models["tinyC"]  # window 24 in layers 0, 2, 3; layer 1 sees everything
    ids = rng.integers(0, cfg["vocab_size"], 60)
    base = P.logits(cfg, w, ids)
    other = ids.copy()
    other[3] = (other[3] + 1) % cfg["vocab_size"]
    assert np.abs(P.logits(cfg, w, other)[-1] - base[-1]).max() > 1e-9  # the full layer still carries it
    # four windowed layers of window 6 reach back at most 4 * 5 tokens
    short = dict(cfg, sliding_window=6, layer_types=["sliding_attention"] * 4)
    a, b = P.logits(short, w, ids), P.logits(short, w, other)
    assert np.array_equal(a[3 + 4 * 5 + 1 :], b[3 + 4 * 5 + 1 :]) and not np.array_equal(a[3 : 3 + 4 * 5 + 1], b[3 : 3 + 4 * 5 + 1])


def test_tied_and_untied_heads(models):
    cfg_a, w_a = models["tinyA"]
    assert cfg_a["tie_word_embeddings"] and w_a["lm_head.weight"] is w_a["model.embed_tokens.weight"]
    cfg_b, w_b = models["tinyB"]
    assert not cfg_b["tie_word_embeddings"] and not np.array_equal(w_b["lm_head.weight"], w_b["model.embed_tokens.weight"])


def test_config_rules():
    cfg = dict(TINY["tinyA"][0])
    del cfg["head_dim"]
    assert P.read_config(cfg)["D"] == 16
    for key, val in (("rope_scaling", {"factor": 2}), ("hidden_act", "gelu")):
        with pytest.raises(NotImplementedError):
            P.read_config(dict(cfg, **{key: val}))


# ------------------------------------------------------------------------------------------ sampling


def test_greedy_takes_the_first_maximum():
    row = np.zeros(40)
    row[[3, 7]] = 5.0
    assert P.sample(row, 0.0, 1, 1) == 3
    row[[30, 5]] = 9.0
    assert P.sample(row, 0.0, 1, 1) == 5


def test_noise_is_uniform_keyed_and_pure():
    u = P.uniform_noise(123, 45, 20000)
    assert u.min() > 0 and u.max() < 1 and abs(u.mean() - 0.5) < 0.01
    assert np.array_equal(u, P.uniform_noise(123, 45, 20000))
    assert not np.array_equal(u, P.uniform_noise(124, 45, 20000)) and not np.array_equal(u, P.uniform_noise(123, 46, 20000))
    assert np.array_equal(u[:100], P.uniform_noise(123, 45, 100))  # entry v does not depend on the vocabulary size
    assert P.mix32(0) == 0 and P.mix32(1) == P.mix32(1) and 0 <= P.mix32(0xFFFFFFFF) < 2**32


def test_temperature_frequencies_follow_softmax():
    logits = np.array([2, 1, 0.5, 0, -1, -3, 1.5, 0.2])
    for temp in (0.5, 2.0):
        draws = [P.sample(logits, temp, seed, 0) for seed in range(4000)]
        freq = np.bincount(draws, minlength=8) / 4000
        p = np.exp(logits / temp)
        assert np.abs(freq - p / p.sum()).max() < 0.03


def test_nucleus_keeps_the_smallest_set_reaching_top_p():
    logits = np.log(np.array([0.5, 0.3, 0.15, 0.05]))
    assert {P.sample(logits, 1.0, s, 0, top_p=0.5) for s in range(300)} == {0}  # mass before token 1 is 0.5, not < 0.5
    assert {P.sample(logits, 1.0, s, 0, top_p=0.6) for s in range(300)} == {0, 1}
    assert {P.sample(logits, 1.0, s, 0, top_p=0.96) for s in range(600)} == {0, 1, 2, 3}
    tie = np.log(np.array([0.25, 0.25, 0.25, 0.25]))
    assert {P.sample(tie, 1.0, s, 0, top_p=0.3) for s in range(300)} == {0, 1}  # ties stay in index order


def test_nucleus_on_the_vectors_of_the_reference_s_sampler_tests():
    """The cases of the reference's tests/test_sampler.py:73-96, with its own numbers: the mass before
    each token of (0.4, 0.3, 0.2, 0.06, 0.04) is 0, 0.4, 0.7, 0.9, 0.96, so top_p 0.8 keeps three and draws
    them in their renormalised shares; a tiny top_p leaves the most likely token whatever the
    temperature; the nucleus goes by probability, not by token id."""
    probs = np.array([0.4, 0.3, 0.2, 0.06, 0.04])
    draws = [P.sample(np.log(probs), 1.0, seed, 0, top_p=0.8) for seed in range(6000)]
    freq = np.bincount(draws, minlength=5) / 6000
    assert freq[3] == 0 and freq[4] == 0
    assert np.abs(freq[:3] - probs[:3] / probs[:3].sum()).max() < 0.025
    assert {P.sample(np.array([0.1, 2.0, 1.9, -1.0]), 3.0, seed, 0, top_p=1e-6) for seed in range(500)} == {1}
    shuffled = np.array([0.04, 0.2, 0.06, 0.4, 0.3])
    seen = np.bincount([P.sample(np.log(shuffled), 1.0, seed, 0, top_p=0.8) for seed in range(3000)], minlength=5)
    assert seen[0] == 0 and seen[2] == 0 and (seen[[1, 3, 4]] > 0).all()


def test_a_draw_depends_on_its_seed_and_position_alone():
    """tests/test_sampler.py:101-113 of the reference: a row's sample is a function of (seed, counter,
    logits); here also of nothing else in the call (the vocabulary's other rows do not exist for it)."""
    r = np.random.default_rng(1)
    for trial in range(20):
        row = r.standard_normal(1000)
        a = P.sample(row, 1.0, 1000 + trial, trial, top_p=0.9)
        assert a == P.sample(row.copy(), 1.0, 1000 + trial, trial, top_p=0.9)
        others = {P.sample(row, 1.0, 1000 + trial, trial + k, top_p=0.9) for k in range(1, 40)}
        assert len(others) > 1  # another position draws other noise


# ------------------------------------------------------------------------------------------ wiring of a layer
#
# What the part tests above cannot see: which norm feeds which product, where the per-head norms sit
# relative to the rotation, which of q_norm / k_norm scales which side, where the residual sums and
# the final norm sit. The library model the reference's own tests compare with is not used here (an
# installed package's model code is no source for this build), so the wiring is pinned by a special
# case worked out independently, in complex arithmetic, and by what must follow from zeroed weights.


def _wiring_config(hidden, layers=1, heads=1, kv_heads=1, inter=8, vocab=None, theta=50.0, eps=1e-6):
    return {"architectures": ["Qwen3ForCausalLM"], "hidden_size": hidden, "intermediate_size": inter,
            "vocab_size": vocab or hidden, "num_hidden_layers": layers, "num_attention_heads": heads,
            "num_key_value_heads": kv_heads, "head_dim": hidden // heads, "rms_norm_eps": eps, "rope_theta": theta,
            "tie_word_embeddings": False, "max_position_embeddings": 64}


def _random_weights(cfg, seed):
    r = np.random.default_rng(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    w = {"model.embed_tokens.weight": r.standard_normal((V, H)), "lm_head.weight": r.standard_normal((V, H)) * 0.3,
         "model.norm.weight": r.uniform(0.5, 1.5, H)}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = r.uniform(0.5, 1.5, H)
        w[p + "post_attention_layernorm.weight"] = r.uniform(0.5, 1.5, H)
        w[p + "self_attn.q_proj.weight"] = r.standard_normal((Hq * D, H)) * 0.4
        w[p + "self_attn.k_proj.weight"] = r.standard_normal((Hkv * D, H)) * 0.4
        w[p + "self_attn.v_proj.weight"] = r.standard_normal((Hkv * D, H)) * 0.4
        w[p + "self_attn.o_proj.weight"] = r.standard_normal((H, Hq * D)) * 0.4
        w[p + "self_attn.q_norm.weight"] = r.uniform(0.3, 1.7, D)
        w[p + "self_attn.k_norm.weight"] = r.uniform(0.3, 1.7, D)
        w[p + "mlp.gate_proj.weight"] = r.standard_normal((I, H)) * 0.4
        w[p + "mlp.up_proj.weight"] = r.standard_normal((I, H)) * 0.4
        w[p + "mlp.down_proj.weight"] = r.standard_normal((H, I)) * 0.4
    return w


def test_one_layer_with_identity_projections_in_closed_form():
    """One layer, one head of the model's width, q/k/v/o projections the identity, no feed-forward
    output, head the identity: the logits are ``norm_f(e_t + sum_s softmax_s(score_ts) x_s)`` with
    ``x = norm_in(e)``. Pairs (j, j + D/2) are complex numbers ``z_j``; the per-head norms scale them
    componentwise *before* the turn by ``exp(i pos theta_j)``, so the score of query t and key s is
    ``Re sum_j a_tj conj(b_sj) exp(i (t - s) theta_j) / sqrt(D)`` with ``a = wq * rmsnorm(x_t)``,
    ``b = wk * rmsnorm(x_s)``. Swapping q_norm and k_norm, norming after the turn, a missing or doubled
    norm, post-norm instead of pre-norm or a wrong scale all change the result (the weights differ
    between the two halves of a pair and between q and k)."""
    D, T, eps, theta = 8, 6, 1e-6, 50.0
    cfg = _wiring_config(D, theta=theta, eps=eps)
    w = _random_weights(cfg, 5)
    p = "model.layers.0."
    eye = np.eye(D)
    for n in ("q", "k", "v", "o"):
        w[p + f"self_attn.{n}_proj.weight"] = eye
    w[p + "mlp.down_proj.weight"] = np.zeros_like(w[p + "mlp.down_proj.weight"])
    w["lm_head.weight"] = eye
    ids = [3, 1, 4, 1, 5, 2]
    got = P.logits(cfg, w, ids)

    def unit(v):  # rmsnorm without a weight
        return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)

    e = w["model.embed_tokens.weight"][ids]
    x = unit(e) * w[p + "input_layernorm.weight"]
    a = unit(x) * w[p + "self_attn.q_norm.weight"]
    b = unit(x) * w[p + "self_attn.k_norm.weight"]
    half = D // 2
    az, bz = a[:, :half] + 1j * a[:, half:], b[:, :half] + 1j * b[:, half:]
    freq = theta ** (-np.arange(half) * 2.0 / D)
    want = np.empty((T, D))
    for t in range(T):
        s = np.arange(t + 1)
        turn = np.exp(1j * (t - s)[:, None] * freq[None, :])
        score = (az[t][None, :] * np.conj(bz[s]) * turn).sum(-1).real / np.sqrt(D)
        prob = np.exp(score - score.max())
        prob /= prob.sum()
        h = e[t] + prob @ x[s]
        want[t] = unit(h) * w["model.norm.weight"]
    assert np.abs(got - want).max() < 1e-5  # float32 angles in the plain implementation
    # the pins bite: swapped per-head norm weights give other logits
    w2 = dict(w)
    w2[p + "self_attn.q_norm.weight"], w2[p + "self_attn.k_norm.weight"] = w[p + "self_attn.k_norm.weight"], w[p + "self_attn.q_norm.weight"]
    assert np.abs(P.logits(cfg, w2, ids) - want).max() > 1e-3


def test_zeroed_weights_say_which_norm_feeds_what():
    cfg = _wiring_config(12, layers=3, heads=3, kv_heads=1, inter=10, vocab=17)
    w = _random_weights(cfg, 6)
    ids = [5, 16, 0, 3, 9, 9, 2]
    base = P.logits(cfg, w, ids)

    # (1) without the mixer's input nothing moves between positions: every position's logits are those of
    # its token alone. If the other norm fed the attention, or the attention read the raw stream, they would mix.
    w1 = dict(w)
    for i in range(3):
        w1[f"model.layers.{i}.input_layernorm.weight"] = np.zeros(12)
    alone = np.stack([P.logits(cfg, w1, [t])[0] for t in ids])
    assert np.abs(P.logits(cfg, w1, ids) - alone).max() < 1e-12 and np.abs(base - alone).max() > 1e-2

    # (2) without the feed-forward's input, its weights do not matter; the attention's still do
    w2 = dict(w)
    for i in range(3):
        w2[f"model.layers.{i}.post_attention_layernorm.weight"] = np.zeros(12)
    ref = P.logits(cfg, w2, ids)
    w2b = dict(w2)
    for i in range(3):
        for n in ("gate", "up", "down"):
            w2b[f"model.layers.{i}.mlp.{n}_proj.weight"] = w2[f"model.layers.{i}.mlp.{n}_proj.weight"] * -3.0 + 1.0
    assert np.abs(P.logits(cfg, w2b, ids) - ref).max() < 1e-12
    w2c = dict(w2)
    w2c["model.layers.1.self_attn.o_proj.weight"] = w2["model.layers.1.self_attn.o_proj.weight"] * 2.0
    assert np.abs(P.logits(cfg, w2c, ids) - ref).max() > 1e-3

    # (3) pre-norm: the stream itself is never normalised. With every o_proj and down_proj zero the logits
    # are the head over the final norm of the bare embedding.
    w3 = dict(w)
    for i in range(3):
        w3[f"model.layers.{i}.self_attn.o_proj.weight"] = np.zeros((12, 12))
        w3[f"model.layers.{i}.mlp.down_proj.weight"] = np.zeros((12, 10))
    e = w["model.embed_tokens.weight"][ids]
    bare = e / np.sqrt((e * e).mean(-1, keepdims=True) + 1e-6) * w["model.norm.weight"] @ w["lm_head.weight"].T
    assert np.abs(P.logits(cfg, w3, ids) - bare).max() < 1e-12

    # (4) the final norm's weight multiplies what the head reads: logits are linear in it, and zero with it
    w4 = dict(w)
    w4["model.norm.weight"] = w["model.norm.weight"] * 2.5
    assert np.allclose(P.logits(cfg, w4, ids), 2.5 * base, rtol=1e-12)
    w4["model.norm.weight"] = np.zeros(12)
    assert np.abs(P.logits(cfg, w4, ids)).max() == 0

    # (5) q and k are normalised per head (their projections' scale does not matter as eps -> 0), v is not
    cfg5 = dict(cfg, rms_norm_eps=1e-30)
    w5 = dict(w)
    base5 = P.logits(cfg5, w, ids)
    for n in ("q", "k"):
        w5[f"model.layers.1.self_attn.{n}_proj.weight"] = w[f"model.layers.1.self_attn.{n}_proj.weight"] * 7.0
    assert np.abs(P.logits(cfg5, w5, ids) - base5).max() < 1e-9
    w5["model.layers.1.self_attn.v_proj.weight"] = w["model.layers.1.self_attn.v_proj.weight"] * 7.0
    assert np.abs(P.logits(cfg5, w5, ids) - base5).max() > 1e-2

    # (6) a layer's norms are its own: zeroing layer 1's input norm is not the same as zeroing layer 0's
    wa, wb = dict(w), dict(w)
    wa["model.layers.0.input_layernorm.weight"] = np.zeros(12)
    wb["model.layers.1.input_layernorm.weight"] = np.zeros(12)
    assert np.abs(P.logits(cfg, wa, ids) - P.logits(cfg, wb, ids)).max() > 1e-3


def test_hash_in_the_reference_s_own_arithmetic():
    """The noise hash once more, in the arithmetic the reference writes it in: int64 tensors holding
    32-bit values, products masked back to 32 bits (miniserve/engine/sampler.py:29-46); and undone by
    the inverse steps (a multiplication by an odd constant and ``x ^= x >> 16`` are both invertible on
    32 bits), which only works out if every shift, constant and mask is the one meant."""
    mask, mul, golden = 0xFFFFFFFF, 0x45D9F3B, 0x9E3779B9

    def mix_t(x):
        x = ((x >> 16) ^ x) * mul & mask
        x = ((x >> 16) ^ x) * mul & mask
        return (x >> 16) ^ x

    xs = torch.tensor([0, 1, 2, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF, 123456789, 0xDEADBEEF], dtype=torch.int64)
    assert mix_t(xs).tolist() == [P.mix32(int(x)) for x in xs]
    seeds, counters, vocab = torch.tensor([123, 0xFFFFFFFF], dtype=torch.int64), torch.tensor([45, 7], dtype=torch.int64), 3000
    key = mix_t(seeds ^ mix_t(counters))
    v = torch.arange(vocab, dtype=torch.int64) * golden
    h = mix_t((key[:, None] + v[None, :]) & mask)
    u = ((h >> 8).to(torch.float64) + 0.5) * (1.0 / (1 << 24))
    for row, (s, c) in enumerate(((123, 45), (0xFFFFFFFF, 7))):
        assert np.array_equal(u[row].numpy(), P.uniform_noise(s, c, vocab))
    inv = pow(mul, -1, 1 << 32)

    def unmix(y):
        y ^= y >> 16
        y = y * inv & mask
        y ^= y >> 16
        y = y * inv & mask
        return y ^ (y >> 16)

    for x in (0, 1, 0xFFFFFFFF, 987654321, 0x80000001):
        assert unmix(P.mix32(x)) == x
    assert len({P.mix32(x) for x in range(5000)}) == 5000
