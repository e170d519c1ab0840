"""Layer parts: mixers, feed-forwards, norms, position encodings, blocks, the decoder."""

from .attention import Attention
from .base import (CacheSpec, FeedForward, LayerCache, Mixer, Norm, Part, PositionDescriptor,
                   PositionEncoding, StateSpec, TensorSpec)
from .block import PreNormBlock
from .feedforward import GatedMLP
from .model import DecoderModel, LayerCall
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
    "Attention", "CacheSpec", "DecoderModel", "FeedForward", "GatedMLP", "LayerCache",
    "LayerCall", "Mixer", "NoPosition", "Norm", "Part", "PositionDescriptor", "PositionEncoding",
    "PreNormBlock",
    "RMSNorm", "RotaryPosition", "StateSpec", "TensorSpec", "build_part", "known",
    "register_block", "register_ffn", "register_mixer", "register_norm", "register_position",
]
