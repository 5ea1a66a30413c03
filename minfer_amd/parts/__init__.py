from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Block, FeedForward, Mixer, Norm,
                   Part, PositionEncoding, Runtime, make_part, register_block, register_feed_forward,
                   register_mixer, register_norm, register_position)
from .spec import BlockSpec, ModelSpec, PartSpec, RunEntry, straight_schedule
from . import attention, block, feedforward, norm, rotary  # registers the built-in parts
from .linear import Linear

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITIONS", "Block", "FeedForward", "Mixer",
           "Norm", "Part", "PositionEncoding", "Runtime", "make_part", "register_block",
           "register_feed_forward", "register_mixer", "register_norm", "register_position",
           "BlockSpec", "ModelSpec", "PartSpec", "RunEntry", "straight_schedule", "Linear"]
