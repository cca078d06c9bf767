from . import attention, block, ends, feedforward, norm, position  # registers the built-in parts
from .base import (Block, Embedding, FeedForward, Head, Mixer, Norm, Part, PositionEncoding,
                   StepContext, build_part, part_class, register_part)

__all__ = ["Block", "Embedding", "FeedForward", "Head", "Mixer", "Norm", "Part",
           "PositionEncoding", "StepContext", "build_part", "part_class", "register_part"]
