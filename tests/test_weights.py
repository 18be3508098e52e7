"""Weights by tensor name: round trip through a model folder, dtypes, the tied head, and the one
error that lists missing and unexpected tensors and wrong shapes (the reference's checks:
tests/test_weights.py:9-48, on its tiny config of hidden 8, inter 16, vocab 32, 2 heads, 1 KV head,
head_dim 4, 2 layers, tied)."""

import json

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

from miniserve_amd.config import config_from_dict
from miniserve_amd.weights import Init, WeightsError, load_weights, random_tensors, write_model_folder
from plain.model_folder import read_model_folder

REF_TINY = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=8, intermediate_size=16, vocab_size=32, num_hidden_layers=2,
    num_attention_heads=2, num_key_value_heads=1, head_dim=4, rms_norm_eps=1e-6, rope_theta=10000.0,
    tie_word_embeddings=True,
)


def spec_of(cfg):
    return config_from_dict(cfg).to_spec()


def test_round_trip_and_tied_head(tmp_path):
    folder = write_model_folder(tmp_path / "m", REF_TINY, seed=0)
    spec = spec_of(REF_TINY)
    w = load_weights(folder, spec, torch.bfloat16, "cpu")
    assert w["lm_head.weight"] is w["model.embed_tokens.weight"]  # the head reads the embedding's tensor itself
    assert all(t.dtype == torch.bfloat16 for t in w.values())
    again = random_tensors(spec, 0)
    assert all(torch.equal(w[k], again[k]) for k in again)
    w32 = load_weights(folder, spec, torch.float32, "cpu")
    assert all(t.dtype == torch.float32 and torch.equal(t, w[k].float()) for k, t in w32.items())
    cfg, plain = read_model_folder(folder)
    assert plain["lm_head.weight"] is plain["model.embed_tokens.weight"]
    assert all(np.array_equal(plain[k], w32[k].double().numpy()) for k in w32)


def test_a_duplicate_head_in_a_tied_checkpoint_is_dropped(tmp_path):
    folder = write_model_folder(tmp_path / "m", REF_TINY, seed=0)
    t = load_file(str(folder / "model.safetensors"))
    t["lm_head.weight"] = torch.zeros(32, 8, dtype=torch.bfloat16)
    save_file(t, str(folder / "model.safetensors"))
    w = load_weights(folder, spec_of(REF_TINY), torch.bfloat16, "cpu")
    assert w["lm_head.weight"] is w["model.embed_tokens.weight"] and float(w["lm_head.weight"].float().abs().max()) > 0


def test_the_loader_follows_whatever_aliases_the_parts_declare(tmp_path):
    """Not the head's private affair: a feed-forward defined here reads a norm weight of another layer under a
    name of its own. Nothing is stored for that name, a stored duplicate is dropped, the name maps to the
    source's tensor itself; an alias of something no part declares is an error when the model is described."""
    import dataclasses

    from miniserve_amd.config import PartSpec
    from miniserve_amd.parts import FeedForward, TensorSpec, register, unregister
    from miniserve_amd.parts.model import expected_aliases, expected_tensors

    @register("feed_forward", "test_scaled")
    class Scaled(FeedForward):
        @classmethod
        def tensors(cls, spec):
            return {"ff.weight": TensorSpec((8, 8))}

        @classmethod
        def aliases(cls, spec):
            return {"ff.scale": spec["scale_from"]}

    try:
        spec = spec_of(REF_TINY)
        layers = list(spec.layers)
        layers[1] = dataclasses.replace(layers[1], feed_forward=PartSpec("test_scaled", {"scale_from": "model.layers.0.input_layernorm.weight"}))
        spec = dataclasses.replace(spec, layers=tuple(layers))
        assert expected_aliases(spec) == {"model.layers.1.ff.scale": "model.layers.0.input_layernorm.weight",
                                          "lm_head.weight": "model.embed_tokens.weight"}
        assert "model.layers.1.ff.scale" not in expected_tensors(spec)
        tensors = random_tensors(spec, 3, Init(0.05, (0.5, 1.5)))
        assert "model.layers.1.ff.scale" not in tensors
        tensors["model.layers.1.ff.scale"] = torch.zeros(8, dtype=torch.bfloat16)  # a duplicate under the alias: dropped
        folder = tmp_path / "m"
        folder.mkdir()
        save_file(tensors, str(folder / "model.safetensors"))
        w = load_weights(folder, spec, torch.bfloat16, "cpu")
        assert w["model.layers.1.ff.scale"] is w["model.layers.0.input_layernorm.weight"]
        bad = dataclasses.replace(spec, layers=(layers[0], dataclasses.replace(layers[1], feed_forward=PartSpec("test_scaled", {"scale_from": "nowhere.weight"}))))
        with pytest.raises(ValueError, match="nowhere.weight"):
            expected_aliases(bad)
    finally:
        unregister("feed_forward", "test_scaled")


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_model_folder(tmp_path / "m", REF_TINY, seed=0)
    f = str(folder / "model.safetensors")
    t = load_file(f)
    del t["model.layers.1.mlp.up_proj.weight"]
    t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(8, dtype=torch.bfloat16)
    t["model.norm.weight"] = torch.ones(9, dtype=torch.bfloat16)
    save_file(t, f)
    with pytest.raises(WeightsError) as e:
        load_weights(folder, spec_of(REF_TINY), torch.bfloat16, "cpu")
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight"]
    assert e.value.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert e.value.mismatched == ["model.norm.weight: (9,) != (8,)"]
    for name in ("up_proj", "q_proj.bias", "model.norm.weight"):
        assert name in str(e.value)
    assert isinstance(e.value, ValueError)


def test_no_safetensors_and_no_config(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(REF_TINY))
    with pytest.raises(FileNotFoundError, match="safetensors"):
        load_weights(tmp_path, spec_of(REF_TINY), torch.bfloat16, "cpu")
    from miniserve_amd.config import load_config

    with pytest.raises(FileNotFoundError, match="config.json"):
        load_config(tmp_path / "nothing")


def test_a_tensor_stored_in_32_bit_stays_32_bit(tmp_path):
    folder = write_model_folder(tmp_path / "m", REF_TINY, seed=0)
    f = str(folder / "model.safetensors")
    t = load_file(f)
    t["model.norm.weight"] = t["model.norm.weight"].float() + 1e-4  # not representable in bfloat16
    t["model.layers.0.mlp.down_proj.weight"] = t["model.layers.0.mlp.down_proj.weight"].to(torch.float16)
    save_file(t, f)
    w = load_weights(folder, spec_of(REF_TINY), torch.bfloat16, "cpu")
    assert w["model.norm.weight"].dtype == torch.float32 and torch.equal(w["model.norm.weight"], t["model.norm.weight"])
    assert w["model.layers.0.mlp.down_proj.weight"].dtype == torch.bfloat16
    assert w["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_an_integer_tensor_is_refused_where_floats_are_expected(tmp_path):
    folder = write_model_folder(tmp_path / "m", REF_TINY, seed=0)
    f = str(folder / "model.safetensors")
    t = load_file(f)
    t["model.norm.weight"] = torch.ones(8, dtype=torch.int64)
    save_file(t, f)
    with pytest.raises(WeightsError, match="model.norm.weight"):
        load_weights(folder, spec_of(REF_TINY), torch.bfloat16, "cpu")


def test_seed_and_init_decide_the_values(tmp_path):
    spec = spec_of(REF_TINY)
    a, b = random_tensors(spec, 1, Init(0.05, (0.5, 1.5))), random_tensors(spec, 2, Init(0.05, (0.5, 1.5)))
    assert not torch.equal(a["model.embed_tokens.weight"], b["model.embed_tokens.weight"])
    n = a["model.norm.weight"].float()
    assert 0.5 <= float(n.min()) and float(n.max()) <= 1.5 and float(n.std()) > 0
    assert float(random_tensors(spec, 1)["model.norm.weight"].float().sub(1).abs().max()) == 0
    e = a["model.embed_tokens.weight"].float()
    assert 0.03 < float(e.std()) < 0.07
