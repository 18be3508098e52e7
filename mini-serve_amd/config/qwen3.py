"""Typed configuration of the Qwen3 dense decoder, read from its own ``config.json`` keys.

Same keys, defaults and refusals as the reference (miniserve/model/qwen3.py:25-55): ``head_dim``
falls back to ``hidden_size // num_attention_heads``; ``rope_scaling`` and an activation other
than ``silu`` are refused. The reference ignores ``architectures``, ``max_position_embeddings``
(its server alone reads it, miniserve/server/__main__.py:29-33) and the sliding-window keys; here
``max_position_embeddings`` is kept as a bound and the window keys select a windowed attention
for the layers they name (parity unpinned: the reference has no window).
"""

from __future__ import annotations

from dataclasses import asdict, dataclass

from .registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry


@register_architecture("Qwen3ForCausalLM")
@dataclass(frozen=True)
class Qwen3Config:
    hidden_size: int
    intermediate_size: int
    vocab_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    max_position_embeddings: int | None = None
    # Per layer: 0 = every earlier key is seen, W > 0 = only the last W keys (itself included).
    layer_windows: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, cfg: dict) -> "Qwen3Config":
        if cfg.get("rope_scaling"):
            raise NotImplementedError(f"rope_scaling={cfg['rope_scaling']!r} is not supported")
        if cfg.get("hidden_act", "silu") != "silu":
            raise NotImplementedError(f"hidden_act={cfg['hidden_act']!r} is not supported")
        if cfg.get("attention_bias"):
            raise NotImplementedError("attention_bias=true is not supported (no bias tensors)")
        missing = [
            k
            for k in (
                "hidden_size",
                "intermediate_size",
                "vocab_size",
                "num_hidden_layers",
                "num_attention_heads",
                "num_key_value_heads",
                "rms_norm_eps",
                "rope_theta",
            )
            if k not in cfg
        ]
        if missing:
            raise KeyError(f"config.json lacks {missing}")
        layers = int(cfg["num_hidden_layers"])
        heads = int(cfg["num_attention_heads"])
        out = cls(
            hidden_size=int(cfg["hidden_size"]),
            intermediate_size=int(cfg["intermediate_size"]),
            vocab_size=int(cfg["vocab_size"]),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=int(cfg["num_key_value_heads"]),
            head_dim=int(cfg.get("head_dim") or cfg["hidden_size"] // heads),
            rms_norm_eps=float(cfg["rms_norm_eps"]),
            rope_theta=float(cfg["rope_theta"]),
            tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
            max_position_embeddings=(
                int(cfg["max_position_embeddings"]) if cfg.get("max_position_embeddings") else None
            ),
            layer_windows=cls._windows(cfg, layers),
        )
        out.validate()
        return out

    @staticmethod
    def _windows(cfg: dict, layers: int) -> tuple[int, ...]:
        """``layer_types`` if given, else ``use_sliding_window`` + ``max_window_layers``: layers
        from index ``max_window_layers`` on attend within ``sliding_window`` keys."""
        window = cfg.get("sliding_window")
        kinds = cfg.get("layer_types")
        if kinds is not None:
            if len(kinds) != layers:
                raise ValueError(f"layer_types has {len(kinds)} entries for {layers} layers")
            known = {"full_attention", "sliding_attention"}
            bad = sorted(set(kinds) - known)
            if bad:
                raise NotImplementedError(f"layer_types {bad} are not supported, expected {sorted(known)}")
            sliding = [k == "sliding_attention" for k in kinds]
        elif cfg.get("use_sliding_window"):
            first = int(cfg.get("max_window_layers", layers))
            sliding = [i >= first for i in range(layers)]
        else:
            sliding = [False] * layers
        if any(sliding) and (not isinstance(window, int) or window < 1):
            raise ValueError(f"sliding-window layers need a positive sliding_window, got {window!r}")
        return tuple(int(window) if s else 0 for s in sliding)

    def validate(self) -> None:
        if min(self.hidden_size, self.intermediate_size, self.vocab_size, self.num_hidden_layers) < 1:
            raise ValueError("sizes must be positive")
        if self.num_attention_heads < 1 or self.num_key_value_heads < 1:
            raise ValueError("head counts must be positive")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ValueError(
                f"num_attention_heads={self.num_attention_heads} is no multiple of "
                f"num_key_value_heads={self.num_key_value_heads}"
            )
        if self.head_dim < 2 or self.head_dim % 2:
            raise ValueError(f"head_dim={self.head_dim} must be even (rotation pairs j with j + head_dim/2)")
        if not self.rms_norm_eps > 0 or not self.rope_theta > 0:
            raise ValueError("rms_norm_eps and rope_theta must be positive")

    def to_dict(self) -> dict:
        """The ``config.json`` that reads back as this configuration."""
        d = asdict(self)
        windows = d.pop("layer_windows")
        d["architectures"] = [self.architecture]
        d["model_type"] = "qwen3"
        d["hidden_act"] = "silu"
        if d["max_position_embeddings"] is None:
            del d["max_position_embeddings"]
        if any(windows):
            sizes = {w for w in windows if w}
            if len(sizes) != 1:
                raise ValueError("config.json holds one sliding_window size")
            d["sliding_window"] = sizes.pop()
            d["layer_types"] = ["sliding_attention" if w else "full_attention" for w in windows]
        return d

    # ------------------------------------------------------------------ lowering

    def to_spec(self) -> ModelSpec:
        h, d = self.hidden_size, self.head_dim
        eps = self.rms_norm_eps

        def norm(tensor: str, width: int) -> PartSpec:
            return PartSpec("rmsnorm", {"width": width, "eps": eps, "tensor": tensor})

        rotary = PartSpec("rotary", {"dim": d, "theta": self.rope_theta})
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = PartSpec(
                "gqa_attention",
                {
                    "prefix": "self_attn.",
                    "hidden_size": h,
                    "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads,
                    "head_dim": d,
                    # Fixed in the reference's code: scale = head_dim ** -0.5 (model/qwen3.py:133-135).
                    "scale": d**-0.5,
                    # QK-RMSNorm is always applied, with the model's one eps (model/qwen3.py:118-119).
                    "qk_norm_eps": eps,
                    "window": self.layer_windows[i] if self.layer_windows else 0,
                    "position": rotary,
                },
            )
            ffn = PartSpec(
                "gated_mlp",
                {"prefix": "mlp.", "hidden_size": h, "intermediate_size": self.intermediate_size, "activation": "silu"},
            )
            block = PartSpec(
                "prenorm",
                {
                    "mixer_norm": norm("input_layernorm.weight", h),
                    "ffn_norm": norm("post_attention_layernorm.weight", h),
                },
            )
            layers.append(LayerSpec(f"model.layers.{i}.", block, mixer, ffn))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=h,
            embedding=PartSpec(
                "token_embedding", {"vocab_size": self.vocab_size, "width": h, "tensor": "model.embed_tokens.weight"}
            ),
            layers=tuple(layers),
            run_order=tuple(RunEntry(i, i) for i in range(self.num_hidden_layers)),
            final_norm=norm("model.norm.weight", h),
            head=PartSpec(
                "linear_head",
                {
                    "vocab_size": self.vocab_size,
                    "width": h,
                    "tensor": "lm_head.weight",
                    "tied_to": "model.embed_tokens.weight" if self.tie_word_embeddings else None,
                },
            ),
            max_position=self.max_position_embeddings,
        )
