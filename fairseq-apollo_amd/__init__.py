"""MI355X-native Mega/Mega2 sequence-mixing path: hand-written HIP kernels (libmega_hip.so,
C ABI in include/mega_hip.h) behind the reference's operator and module surface."""
from . import _lib, ops  # noqa: F401
from .modules import (  # noqa: F401
    AttentionSoftmax,
    BaseMovingLayer,
    EfficientAttention,
    MultiHeadComplexEMA,
    MultiHeadEMA,
    SequenceNorm,
    SwiGLU,
    TimestepNorm,
    norm_then_move,
)

from .layers import (  # noqa: F401,E402
    Mega2Layer,
    MegaDecoderLayer,
    MegaEncoderLayer,
    MovingAverageGatedAttention,
    NormalizedFeedForwardNetwork,
    RMSNorm,
    RotaryEmbedding,
    streamed_forward,
)

from .model import MegaDecoderNoCrossAttn, validate_stream  # noqa: F401,E402

__all__ = [
    "MegaDecoderNoCrossAttn",
    "validate_stream",
    "Mega2Layer",
    "MegaDecoderLayer",
    "MegaEncoderLayer",
    "streamed_forward",
    "MovingAverageGatedAttention",
    "NormalizedFeedForwardNetwork",
    "RMSNorm",
    "RotaryEmbedding",
    "ops",
    "AttentionSoftmax",
    "BaseMovingLayer",
    "EfficientAttention",
    "MultiHeadComplexEMA",
    "MultiHeadEMA",
    "SequenceNorm",
    "SwiGLU",
    "TimestepNorm",
    "norm_then_move",
]
