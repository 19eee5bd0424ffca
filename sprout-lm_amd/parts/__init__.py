from .base import (Block, FeedForward, Mixer, Norm, NormFold, Part, PositionEncoding, make_part, register_part,
                   registered_parts)
from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (register the built-in parts)

__all__ = ["Block", "FeedForward", "Mixer", "Norm", "NormFold", "Part", "PositionEncoding", "make_part", "register_part",
           "registered_parts"]
