from .base import (Block, BranchScale, FeedForward, Mixer, Norm, NormFold, Part, PositionEncoding, make_part, register_part,
                   registered_parts)
from . import attention, block, conv, embedding, latent_attention, mixed_heads_attention, mlp, moe, norm, recurrence, retention, rotary, scale, sink_attention, ssm  # noqa: F401  (register the built-in parts)

__all__ = ["Block", "BranchScale", "FeedForward", "Mixer", "Norm", "NormFold", "Part", "PositionEncoding", "make_part", "register_part",
           "registered_parts"]
