from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (registers the built-in kinds)
from .base import (
    Block, FeedForward, KVCacheSpec, Mixer, Norm, NormHandoff, Part, PositionEncoding, StateSpec, part_class,
    register_block, register_embedding, register_ffn, register_head, register_mixer, register_norm,
    register_position, registered, unregister,
)

__all__ = [
    "Block", "FeedForward", "KVCacheSpec", "Mixer", "Norm", "NormHandoff", "Part", "PositionEncoding", "StateSpec",
    "part_class", "register_block", "register_embedding", "register_ffn", "register_head",
    "register_mixer", "register_norm", "register_position", "registered", "unregister",
]
