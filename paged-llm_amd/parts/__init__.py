"""Parts a decoder layer is put together from; importing this package registers the built-in ones."""
from . import attention, block, embedding, feedforward, latent_attention, moe, norm, normed_attention, parallel, recurrent, rope, stream_ops  # noqa: F401
from .base import BLOCK, Block, CacheSpec, PageTensor, FeedForward, GraphLayout, Mixer, Norm, Part, PositionEncoding, StateSpec, StreamOp
from .registry import (BuildEnv, build, register_block, register_embedding, register_feed_forward, register_head,
                       register_mixer, register_norm, register_position_encoding, register_stream_op)
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleStep, StreamOpSpec, WeightSpec

__all__ = ["BLOCK", "Block", "CacheSpec", "PageTensor", "FeedForward", "GraphLayout", "Mixer", "Norm", "Part", "PositionEncoding", "StateSpec", "BuildEnv",
           "build", "register_block", "register_embedding", "register_feed_forward", "register_head", "register_mixer",
           "register_norm", "register_position_encoding", "register_stream_op", "StreamOp", "StreamOpSpec", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleStep",
           "WeightSpec"]
