"""Parts a decoder layer is put together from; importing this package registers the built-in ones."""
from . import attention, block, embedding, feedforward, norm, rope  # noqa: F401
from .base import BLOCK, Block, CacheSpec, PageTensor, FeedForward, GraphLayout, Mixer, Norm, Part, PositionEncoding, StateSpec
from .registry import (BuildEnv, build, register_block, register_embedding, register_feed_forward, register_head,
                       register_mixer, register_norm, register_position_encoding)
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleStep, WeightSpec

__all__ = ["BLOCK", "Block", "CacheSpec", "PageTensor", "FeedForward", "GraphLayout", "Mixer", "Norm", "Part", "PositionEncoding", "StateSpec", "BuildEnv",
           "build", "register_block", "register_embedding", "register_feed_forward", "register_head", "register_mixer",
           "register_norm", "register_position_encoding", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleStep",
           "WeightSpec"]
