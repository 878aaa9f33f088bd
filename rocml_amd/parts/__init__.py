from .base import (BuildContext, Embedding, FeedForward, Head, KVCacheRequest, Mixer, Norm, ParamSpec, Part,
                   PositionEncoding, StateRequest)
from .registry import (build_block, build_embedding, build_feed_forward, build_head, build_mixer, build_norm,
                       build_position, register_block, register_embedding, register_feed_forward,
                       register_head, register_mixer, register_norm, register_position)
from . import rmsnorm, rope, attention, mlp, block, embedding, head  # noqa: F401  (register the built-in parts)

__all__ = ["BuildContext", "Embedding", "FeedForward", "Head", "KVCacheRequest", "Mixer", "Norm", "ParamSpec",
           "Part", "PositionEncoding", "StateRequest", "build_block", "build_embedding", "build_feed_forward",
           "build_head", "build_mixer", "build_norm", "build_position", "register_block", "register_embedding",
           "register_feed_forward", "register_head", "register_mixer", "register_norm", "register_position"]
