from . import attention, block, embedding, mlp, moe, norm, rope  # noqa: F401  (registration)
from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block,
                   FeedForward, LayerCache, LayerSpec, Mixer, ModelSpec, Norm, ParamSpec, Part, PartSpec,
                   PositionEncoding, Rotary, ScheduleEntry, StepContext, walk_params, walk_parts)

__all__ = ["BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block",
           "FeedForward", "LayerCache", "LayerSpec", "Mixer", "ModelSpec", "Norm", "ParamSpec", "Part", "PartSpec",
           "PositionEncoding", "Rotary", "ScheduleEntry", "StepContext", "walk_params", "walk_parts"]
