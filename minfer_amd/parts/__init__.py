from .base import (BLOCKS, COMBINERS, Combiner, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, Block, Embedding,
                   FeedForward, Head, Mixer, Norm, NormAhead, Normed, Part, PositionEncoding, Runtime, announce_norm,
                   make_part, normed_input, register_block,
                   register_embedding, register_feed_forward, register_head, register_mixer, register_norm,
                   register_position, register_combiner)
from .spec import BlockSpec, ModelSpec, PartSpec, RunEntry, straight_schedule
from . import (attention, block, capped_attention, combine, embedding, feedforward, gated_recurrence,  # registers the built-in parts
               latent_attention, linear_attention, moe, norm, normed_attention, recurrent, rotary, side_by_side)
from .linear import Linear

__all__ = ["BLOCKS", "COMBINERS", "Combiner", "register_combiner", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS", "Block", "Embedding",
           "FeedForward", "Head", "Mixer", "Norm", "NormAhead", "Normed", "Part", "PositionEncoding", "Runtime",
           "announce_norm", "make_part", "normed_input",
           "register_block", "register_embedding", "register_feed_forward", "register_head", "register_mixer",
           "register_norm", "register_position", "BlockSpec", "ModelSpec", "PartSpec", "RunEntry",
           "straight_schedule", "Linear"]
