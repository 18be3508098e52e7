"""Named ``config.json`` dictionaries: two tiny shapes that differ in every size and option, one
tiny windowed shape, and the three benchmark shapes (random weights; no checkpoint is fetched).

The reference names models by size and maps them to pinned downloads
(miniserve/model/weights.py:24-29); without a network the names map to shapes instead.
"""

from __future__ import annotations


def _qwen3(**kw) -> dict:
    base = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu"}
    base.update(kw)
    return base


PRESETS: dict[str, dict] = {
    "tinyA": _qwen3(
        num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
        intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=128,
    ),
    "tinyB": _qwen3(
        num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
        intermediate_size=224, vocab_size=379, rope_theta=1e6, rms_norm_eps=1e-5,
        tie_word_embeddings=False, max_position_embeddings=256,
    ),
    "tinyC": _qwen3(
        num_hidden_layers=4, hidden_size=80, num_attention_heads=3, num_key_value_heads=3, head_dim=48,
        intermediate_size=176, vocab_size=517, rope_theta=50000.0, rms_norm_eps=3e-6,
        tie_word_embeddings=False, max_position_embeddings=512, sliding_window=24,
        layer_types=["sliding_attention", "full_attention", "sliding_attention", "sliding_attention"],
    ),
    # Head sizes 64 and 128 with 16-token pages: the shapes the matrix-core attention kernels take.
    "tinyD": _qwen3(
        num_hidden_layers=2, hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
        intermediate_size=192, vocab_size=300, rope_theta=10000.0, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=2048,
    ),
    "tinyE": _qwen3(
        num_hidden_layers=3, hidden_size=160, num_attention_heads=4, num_key_value_heads=1, head_dim=128,
        intermediate_size=288, vocab_size=411, rope_theta=1e6, rms_norm_eps=1e-5,
        tie_word_embeddings=False, max_position_embeddings=4096, sliding_window=100,
        layer_types=["full_attention", "sliding_attention", "full_attention"],
    ),
    "0.6B": _qwen3(
        num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
        intermediate_size=3072, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=40960,
    ),
    "8B": _qwen3(
        num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
        intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
        tie_word_embeddings=False, max_position_embeddings=40960,
    ),
    "32B": _qwen3(
        num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
        intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
        tie_word_embeddings=False, max_position_embeddings=40960,
    ),
}


def preset(name: str) -> dict:
    try:
        return dict(PRESETS[name])
    except KeyError:
        raise ValueError(f"unknown preset {name!r}, expected one of {sorted(PRESETS)}") from None
