from .registry import (
    ARCHITECTURES,
    architecture_name,
    config_from_dict,
    load_config,
    load_config_dict,
    register_architecture,
    unregister_architecture,
)
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from .qwen3 import Qwen3Config
from .presets import PRESETS, preset

__all__ = [
    "ARCHITECTURES", "architecture_name", "config_from_dict", "load_config", "load_config_dict",
    "register_architecture", "unregister_architecture", "LayerSpec", "ModelSpec", "PartSpec",
    "RunEntry", "Qwen3Config", "PRESETS", "preset",
]
