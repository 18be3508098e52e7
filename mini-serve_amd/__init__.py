"""A small single-GPU inference engine for MI355X (gfx950): typed configuration and registry,
weights by tensor name, layers composed from parts, a paged cache manager, one step function, a
continuous-batching scheduler, on-device sampling, and hand-written HIP kernels underneath."""

from . import parts as _parts  # noqa: F401  registers the built-in parts
from .config import PRESETS, Qwen3Config, config_from_dict, load_config, preset, register_architecture

__all__ = ["PRESETS", "Qwen3Config", "config_from_dict", "load_config", "preset", "register_architecture"]
__version__ = "0.1.0"
