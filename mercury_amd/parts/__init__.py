"""Layer parts: mixers, feed-forwards, norms, position encodings, blocks, the decoder."""

from .attention import Attention
from .base import (CacheSpec, FeedForward, LayerCache, Mixer, Norm, Part, PositionDescriptor,
                   PositionEncoding, StateSpec, TensorSpec)
from .block import PreNormBlock
from .embedding import OutputHead, TokenEmbedding
from .feedforward import GatedMLP
from .lowering import OneOp
from .model import CallerStep, DecoderModel, LayerCall, Registers
from .norm import RMSNorm
from .position import NoPosition, RotaryPosition
from .registry import (build_part, known, register_block, register_ffn, register_mixer,
                       register_norm, register_position)

register_mixer("attention")(Attention)
register_ffn("gated_mlp")(GatedMLP)
register_norm("rmsnorm")(RMSNorm)
register_position("rotary")(RotaryPosition)
register_position("none")(NoPosition)
register_block("pre_norm")(PreNormBlock)

__all__ = [
    "Attention", "CacheSpec", "CallerStep", "DecoderModel", "FeedForward", "GatedMLP",
    "LayerCache", "LayerCall", "Mixer", "NoPosition", "Norm", "OneOp", "OutputHead", "Part",
    "PositionDescriptor", "PositionEncoding", "PreNormBlock", "Registers",
    "RMSNorm", "RotaryPosition", "StateSpec", "TensorSpec", "TokenEmbedding", "build_part", "known",
    "register_block", "register_ffn", "register_mixer", "register_norm", "register_position",
]
