from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (register the built-in parts)
from .base import (
    Block, CachePlane, Embedding, FeedForward, Head, KVNeed, Mixer, Norm, Part, PositionEncoding, Rotation,
    Runtime, StateNeed, StateTensor, TensorSpec,
)
from .model import CacheSlotNeed, DecoderModel, expected_tensors
from .registry import PARTS, part_class, register, unregister

__all__ = [
    "Block", "CachePlane", "Embedding", "FeedForward", "Head", "KVNeed", "Mixer", "Norm", "Part",
    "PositionEncoding", "Rotation", "Runtime", "StateNeed", "StateTensor", "TensorSpec", "CacheSlotNeed",
    "DecoderModel", "expected_tensors", "PARTS", "part_class", "register", "unregister",
]
