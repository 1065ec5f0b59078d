from pyre_amd.parts.base import (AttentionSpec, BlockSpec, EmbeddingSpec, FeedForward,
                                 LayerCall, LMHeadSpec, Mixer, ModelSpec, Norm, NoPositionSpec, Part,
                                 PagedCacheSpec, PagedTensorSpec, PositionEncoding, RMSNormSpec, RotarySpec, StateCacheSpec, SwiGLUSpec,
                                 TensorSpec, make_part, register_part)

__all__ = ["AttentionSpec", "BlockSpec", "EmbeddingSpec", "FeedForward", "LayerCall",
           "LMHeadSpec", "Mixer", "ModelSpec", "Norm", "NoPositionSpec", "PagedCacheSpec", "PagedTensorSpec", "Part", "PositionEncoding",
           "RMSNormSpec", "RotarySpec", "StateCacheSpec", "SwiGLUSpec", "TensorSpec", "make_part",
           "register_part"]
