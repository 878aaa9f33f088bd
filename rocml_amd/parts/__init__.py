from .base import (BuildContext, FeedForward, KVCacheRequest, Mixer, Norm, ParamSpec, Part,
                   PositionEncoding, StateRequest)
from .registry import (build_block, build_feed_forward, build_mixer, build_norm, build_position,
                       register_block, register_feed_forward, register_mixer, register_norm,
                       register_position)
from . import rmsnorm, rope, attention, mlp, block  # noqa: F401  (register the built-in parts)

__all__ = ["BuildContext", "FeedForward", "KVCacheRequest", "Mixer", "Norm", "ParamSpec", "Part",
           "PositionEncoding", "StateRequest", "build_block", "build_feed_forward", "build_mixer",
           "build_norm", "build_position", "register_block", "register_feed_forward",
           "register_mixer", "register_norm", "register_position"]
