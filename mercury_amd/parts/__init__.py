"""Layer parts: mixers, feed-forwards, norms, position encodings, blocks, the decoder."""

from .attention import Attention
from .base import (CacheSpec, FeedForward, LayerCache, Mixer, Norm, Part, PositionDescriptor,
                   PositionEncoding, StateSpec, TensorSpec)
from .block import ParallelBlock, PreNormBlock, PrePostNormBlock
from .embedding import OutputHead, TokenEmbedding
from .experts import RoutedExperts
from .feedforward import GatedMLP, UnaryMLP
from .latent_attention import LatentAttention
from .lowering import OneOp
from .mixer_sum import NormedMixerSum
from .model import CallerStep, DecoderModel, LayerCall, Registers
from .mlstm import MatrixMemory
from .norm import NoNorm, RMSNorm
from .position import NoPosition, RotaryPosition
from .state_space import StateSpaceMixer
from .stream_mix import StreamMix
from .retention import Retention
from .registry import (build_part, known, register_block, register_ffn, register_mixer,
                       register_norm, register_position)

register_mixer("attention")(Attention)
register_mixer("latent_attention")(LatentAttention)
register_ffn("gated_mlp")(GatedMLP)
register_ffn("routed_experts")(RoutedExperts)
register_ffn("unary_mlp")(UnaryMLP)
register_mixer("state_space")(StateSpaceMixer)
register_mixer("normed_sum")(NormedMixerSum)
register_mixer("retention")(Retention)
register_mixer("matrix_memory")(MatrixMemory)
register_norm("rmsnorm")(RMSNorm)
register_norm("none")(NoNorm)
register_position("rotary")(RotaryPosition)
register_position("none")(NoPosition)
register_block("pre_norm")(PreNormBlock)
register_block("parallel")(ParallelBlock)
register_block("pre_post_norm")(PrePostNormBlock)

__all__ = [
    "Attention", "CacheSpec", "CallerStep", "DecoderModel", "FeedForward", "GatedMLP",
    "LatentAttention", "LayerCache", "LayerCall", "MatrixMemory", "Mixer", "NoNorm", "NoPosition", "Norm", "OneOp", "OutputHead", "Part",
    "ParallelBlock", "PositionDescriptor", "PrePostNormBlock", "Retention", "PositionEncoding", "PreNormBlock", "Registers",
    "RoutedExperts", "NormedMixerSum", "StateSpaceMixer", "StreamMix", "UnaryMLP",
    "RMSNorm", "RotaryPosition", "StateSpec", "TensorSpec", "TokenEmbedding", "build_part", "known",
    "register_block", "register_ffn", "register_mixer", "register_norm", "register_position",
]
