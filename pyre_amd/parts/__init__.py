from pyre_amd.parts.base import (AttentionSpec, BlockSpec, EmbeddingSpec, FeedForward, KVCacheSpec,
                                 LayerCall, LMHeadSpec, Mixer, ModelSpec, Norm, NoPositionSpec, Part,
                                 PositionEncoding, RMSNormSpec, RotarySpec, StateCacheSpec, SwiGLUSpec,
                                 TensorSpec, make_part, register_part)

__all__ = ["AttentionSpec", "BlockSpec", "EmbeddingSpec", "FeedForward", "KVCacheSpec", "LayerCall",
           "LMHeadSpec", "Mixer", "ModelSpec", "Norm", "NoPositionSpec", "Part", "PositionEncoding",
           "RMSNormSpec", "RotarySpec", "StateCacheSpec", "SwiGLUSpec", "TensorSpec", "make_part",
           "register_part"]
