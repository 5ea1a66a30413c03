from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, Block, Embedding,
                   FeedForward, Head, Mixer, Norm, NormAhead, Normed, Part, PositionEncoding, Runtime, announce_norm,
                   make_part, normed_input, register_block,
                   register_embedding, register_feed_forward, register_head, register_mixer, register_norm,
                   register_position)
from .spec import BlockSpec, ModelSpec, PartSpec, RunEntry, straight_schedule
from . import attention, block, embedding, feedforward, norm, rotary  # registers the built-in parts
from .linear import Linear

__all__ = ["BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS", "Block", "Embedding",
           "FeedForward", "Head", "Mixer", "Norm", "NormAhead", "Normed", "Part", "PositionEncoding", "Runtime",
           "announce_norm", "make_part", "normed_input",
           "register_block", "register_embedding", "register_feed_forward", "register_head", "register_mixer",
           "register_norm", "register_position", "BlockSpec", "ModelSpec", "PartSpec", "RunEntry",
           "straight_schedule", "Linear"]
