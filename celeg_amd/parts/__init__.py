from .base import (Part, Norm, Mixer, FeedForward, PositionEncoding, Embedding, Head,
                   WeightSpec, KVNeed, StateNeed, Runtime, register_part, build_part,
                   build_block, registered_parts)
from . import norm, position, attention, short_conv, feed_forward, embedding, block  # noqa: F401

__all__ = ["Part", "Norm", "Mixer", "FeedForward", "PositionEncoding", "Embedding", "Head",
           "WeightSpec", "KVNeed", "StateNeed", "Runtime", "register_part", "build_part", "build_block",
           "registered_parts"]
