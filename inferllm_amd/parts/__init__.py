from . import (attention, block, delta_rule, ends, feedforward, latent_attention, norm, position,  # registers
               recurrent, side_by_side)                                                                   # the built-in parts
from .base import (Block, Embedding, FeedForward, Head, Mixer, Norm, Part, PositionEncoding,
                   StepContext, build_part, part_class, register_part)

__all__ = ["Block", "Embedding", "FeedForward", "Head", "Mixer", "Norm", "Part",
           "PositionEncoding", "StepContext", "build_part", "part_class", "register_part"]
