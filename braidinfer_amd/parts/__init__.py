from .base import (Part, Norm, NormedInput, ResidualSink, PositionEncoding, RotaryTables, Mixer, MixerContext, FeedForward, Embedding,
                   OutputHead, Runtime, register_part, unregister_part, build_part, block_arrangement,
                   registered_parts)
from . import norm, rope, attention, feedforward, embedding, block  # noqa: F401  (register the built-in parts)
from .linear import linear, fuse_rows

__all__ = ["Part", "Norm", "NormedInput", "ResidualSink", "PositionEncoding", "RotaryTables", "Mixer", "MixerContext", "FeedForward",
           "Embedding", "OutputHead", "Runtime", "register_part", "unregister_part", "build_part",
           "block_arrangement", "registered_parts", "linear", "fuse_rows"]
