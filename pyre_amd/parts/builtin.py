"""Registers the parts that ship with the framework."""

from pyre_amd.parts.attention import Attention
from pyre_amd.parts.base import register_part
from pyre_amd.parts.block import PreNormBlock
from pyre_amd.parts.embedding import LMHead, TokenEmbedding
from pyre_amd.parts.feedforward import SwiGLU
from pyre_amd.parts.norm import RMSNorm
from pyre_amd.parts.rotary import NoPosition, RotaryEncoding

register_part("mixer", "attention", Attention)
register_part("feed_forward", "swiglu", SwiGLU)
register_part("norm", "rmsnorm", RMSNorm)
register_part("position", "rotary", RotaryEncoding)
register_part("position", "none", NoPosition)
register_part("block", "pre_norm", PreNormBlock)
register_part("embedding", "embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)
