from .base import (Arena, FeedForward, KVNeed, Mixer, Norm, PositionEncoding, StateNeed, StepContext,
                   build_feed_forward, build_mixer, build_norm, build_position, register_feed_forward,
                   register_mixer, register_norm, register_position, to_matrix, to_vector)
from . import norms, positions, attention, feedforward  # noqa: F401  (register the built-in kinds)
from .block import Block

__all__ = ["Arena", "Block", "FeedForward", "KVNeed", "Mixer", "Norm", "PositionEncoding", "StateNeed",
           "StepContext", "build_feed_forward", "build_mixer", "build_norm", "build_position",
           "register_feed_forward", "register_mixer", "register_norm", "register_position",
           "to_matrix", "to_vector"]
