from .base import (CacheNeed, FeedForward, Mixer, Norm, NormedRows, Part, PositionEncoding, RotaryTable, Runtime, StateNeed,
                   Transform, WeightWant, Workspace, make, register_block, register_feed_forward, register_mixer,
                   register_norm, register_position, register_transform)
from .model import DecoderModel
from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec

__all__ = [
    "CacheNeed", "DecoderModel", "FeedForward", "LayerRun", "LayerSpec", "Mixer", "ModelSpec", "Norm", "Part",
    "NormedRows", "PartSpec", "PositionEncoding", "RotaryTable", "Runtime", "StateNeed", "Transform", "WeightWant", "Workspace",
    "make", "register_block", "register_feed_forward", "register_mixer", "register_norm", "register_position",
    "register_transform",
]
