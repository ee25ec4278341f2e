from .base import (Block, CacheBinding, CacheSpec, FeedForward, Mixer, Norm, Part, PositionEncoding, StateSpec,
                   TensorDecl, build_block, build_part, register_block, register_embedding, register_feed_forward,
                   register_head, register_mixer, register_norm, register_position)
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registers the built-in parts)

__all__ = ["Block", "CacheBinding", "CacheSpec", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding",
           "StateSpec", "TensorDecl", "build_block", "build_part", "register_block", "register_embedding",
           "register_feed_forward", "register_head", "register_mixer", "register_norm", "register_position"]
