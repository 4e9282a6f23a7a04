from .base import (Block, BranchScale, FeedForward, Mixer, Norm, NormFold, Part, PositionEncoding, make_part, register_part,
                   registered_parts)
from . import attention, block, embedding, latent_attention, mlp, moe, norm, recurrence, retention, rotary, scale, sink_attention  # noqa: F401  (register the built-in parts)

__all__ = ["Block", "BranchScale", "FeedForward", "Mixer", "Norm", "NormFold", "Part", "PositionEncoding", "make_part", "register_part",
           "registered_parts"]
