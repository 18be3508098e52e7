"""Configuration and registry: keys, defaults and refusals of the typed configuration
(the reference's: miniserve/model/qwen3.py:38-55, tests/test_consistency.py:148-151), the lowering
to a model description, and the architecture registry."""

import pytest

from miniserve_amd.config import (
    ARCHITECTURES, ModelSpec, PartSpec, Qwen3Config, RunEntry, config_from_dict, preset, register_architecture,
    unregister_architecture,
)
from miniserve_amd.parts import expected_tensors


def test_reads_its_own_keys():
    c = config_from_dict(preset("tinyB"))
    assert isinstance(c, Qwen3Config)
    assert (c.hidden_size, c.intermediate_size, c.vocab_size, c.num_hidden_layers) == (96, 224, 379, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (6, 1, 32)
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 1e6 and c.tie_word_embeddings is False


def test_head_dim_defaults_to_hidden_over_heads():
    d = preset("tinyA")
    del d["head_dim"]
    assert config_from_dict(d).head_dim == 64 // 4
    d["head_dim"] = None
    assert config_from_dict(d).head_dim == 16


def test_refusals():
    for key, val in (("rope_scaling", {"type": "yarn", "factor": 2.0}), ("hidden_act", "gelu"), ("attention_bias", True)):
        d = preset("tinyA")
        d[key] = val
        with pytest.raises(NotImplementedError, match=key):
            config_from_dict(d)
    d = preset("tinyA")
    d["num_key_value_heads"] = 3
    with pytest.raises(ValueError, match="multiple"):
        config_from_dict(d)
    d = preset("tinyA")
    del d["rms_norm_eps"]
    with pytest.raises(KeyError, match="rms_norm_eps"):
        config_from_dict(d)


def test_unknown_architecture_lists_known_ones():
    d = preset("tinyA")
    d["architectures"] = ["LlamaForCausalLM"]
    with pytest.raises(ValueError, match="Qwen3ForCausalLM"):
        config_from_dict(d)
    del d["architectures"]
    with pytest.raises(ValueError, match="architectures"):
        config_from_dict(d)


def test_windows_from_either_spelling():
    d = preset("tinyA")
    d.update(use_sliding_window=True, sliding_window=8, max_window_layers=1)
    assert config_from_dict(d).layer_windows == (0, 8)
    d = preset("tinyC")
    assert config_from_dict(d).layer_windows == (24, 0, 24, 24)
    d["sliding_window"] = None
    with pytest.raises(ValueError, match="sliding_window"):
        config_from_dict(d)
    # the keys alone switch nothing on
    d = preset("tinyA")
    d.update(sliding_window=8, max_window_layers=1)
    assert config_from_dict(d).layer_windows == (0, 0)


def test_round_trip_through_config_json():
    for name in ("tinyA", "tinyB", "tinyC", "0.6B"):
        c = config_from_dict(preset(name))
        assert config_from_dict(c.to_dict()) == c


def test_lowering_holds_every_constant():
    c = config_from_dict(preset("tinyC"))
    s = c.to_spec()
    assert len(s.layers) == 4 and [e.layer for e in s.run_order] == [0, 1, 2, 3]
    m = s.layers[2].mixer
    assert m.kind == "gqa_attention" and m["window"] == 24 and m["scale"] == 48**-0.5 and m["qk_norm_eps"] == 3e-6
    assert m["position"].kind == "rotary" and m["position"]["theta"] == 50000.0 and m["position"]["dim"] == 48
    assert s.layers[1].mixer["window"] == 0
    assert s.layers[0].feed_forward["intermediate_size"] == 176
    assert s.final_norm["eps"] == 3e-6 and s.head["tied_to"] is None
    assert config_from_dict(preset("tinyA")).to_spec().head["tied_to"] == "model.embed_tokens.weight"


def test_expected_tensors_match_the_reference_names():
    names = expected_tensors(config_from_dict(preset("tinyB")).to_spec())
    p = "model.layers.2."
    for n, shape in {
        "model.embed_tokens.weight": (379, 96), "model.norm.weight": (96,), "lm_head.weight": (379, 96),
        p + "input_layernorm.weight": (96,), p + "post_attention_layernorm.weight": (96,),
        p + "self_attn.q_proj.weight": (192, 96), p + "self_attn.k_proj.weight": (32, 96),
        p + "self_attn.v_proj.weight": (32, 96), p + "self_attn.o_proj.weight": (96, 192),
        p + "self_attn.q_norm.weight": (32,), p + "self_attn.k_norm.weight": (32,),
        p + "mlp.gate_proj.weight": (224, 96), p + "mlp.up_proj.weight": (224, 96), p + "mlp.down_proj.weight": (96, 224),
    }.items():
        assert names[n].shape == shape, n
    assert len(names) == 3 + 3 * 11
    assert "lm_head.weight" not in expected_tensors(config_from_dict(preset("tinyA")).to_spec())


def test_run_order_is_data():
    layer = config_from_dict(preset("tinyA")).to_spec().layers[0]
    base = dict(architecture="X", vocab_size=8, hidden_size=64, embedding=PartSpec("token_embedding"), layers=(layer,),
                final_norm=PartSpec("rmsnorm"), head=PartSpec("linear_head"))
    twice = ModelSpec(run_order=(RunEntry(0, 0), RunEntry(0, 1)), **base)  # one layer's weights run twice
    assert twice.num_cache_slots == 2
    shared = ModelSpec(run_order=(RunEntry(0, 0), RunEntry(0, 0, writes_cache=False)), **base)  # reads the other's cache
    assert shared.num_cache_slots == 1
    with pytest.raises(ValueError, match="written by two"):
        ModelSpec(run_order=(RunEntry(0, 0), RunEntry(0, 0)), **base)
    with pytest.raises(ValueError, match="before any entry wrote"):
        ModelSpec(run_order=(RunEntry(0, 0, writes_cache=False),), **base)
    with pytest.raises(ValueError, match="names layer"):
        ModelSpec(run_order=(RunEntry(1, 0),), **base)


def test_registering_an_architecture():
    @register_architecture("ToyForCausalLM")
    class ToyConfig:
        @classmethod
        def from_dict(cls, cfg):
            return cls()

    try:
        assert isinstance(config_from_dict({"architectures": ["ToyForCausalLM"]}), ToyConfig)
        with pytest.raises(ValueError, match="already registered"):
            register_architecture("ToyForCausalLM")(type("Other", (), {}))
    finally:
        unregister_architecture("ToyForCausalLM")
    assert "ToyForCausalLM" not in ARCHITECTURES


def test_head_sizes_the_kernels_refuse_are_refused_when_the_model_is_built():
    """Not in the first step: the attention part checks its head shape when it is constructed."""
    from miniserve_amd.config.spec import PartSpec
    from miniserve_amd.parts.attention import GQAttention

    def spec(**kw):
        base = dict(hidden_size=64, num_heads=4, num_kv_heads=2, head_dim=16, scale=0.25)
        base.update(kw)
        return PartSpec("gqa_attention", base)

    GQAttention(spec(), None)
    for bad in (24, 8, 272, 100):
        with pytest.raises(ValueError, match="head_dim"):
            GQAttention(spec(head_dim=bad), None)
    with pytest.raises(ValueError, match="no multiple"):
        GQAttention(spec(num_heads=5), None)
    with pytest.raises(ValueError, match="scale"):
        GQAttention(spec(scale=0.0), None)
