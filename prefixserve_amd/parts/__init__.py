from .base import (CacheNeed, FeedForward, Mixer, Norm, NormedRows, Part, PositionEncoding, RotaryTable, Runtime, StateNeed,
                   WeightWant, Workspace, make, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position)
from .model import DecoderModel
from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec

__all__ = [
    "CacheNeed", "DecoderModel", "FeedForward", "LayerRun", "LayerSpec", "Mixer", "ModelSpec", "Norm", "Part",
    "PartSpec", "PositionEncoding", "RotaryTable", "Runtime", "StateNeed", "WeightWant", "Workspace", "make", "register_block",
    "register_feed_forward", "register_mixer", "register_norm", "register_position",
]
