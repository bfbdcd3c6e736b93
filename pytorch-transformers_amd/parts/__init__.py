"""Parts that models are put together from: mixers, feed-forwards, norms, position encodings, blocks."""
from .base import Part, StepContext, make_part, register_part, registered_parts
from .linear import Embedding, Linear, OutputHead, QkvTail, TailDone
from .norms import LayerNorm
from .positions import AlibiPositions, NoPositions, Rotation, RotaryPositions, ScoreBias, alibi_slopes
from .attention import AttentionMixer
from .feedforward import DenseFeedForward
from .blocks import ParallelBlock, SequentialBlock

__all__ = ["Part", "StepContext", "make_part", "register_part", "registered_parts", "Embedding", "Linear",
           "OutputHead", "LayerNorm", "AlibiPositions", "NoPositions", "Rotation", "RotaryPositions", "ScoreBias", "alibi_slopes",
           "AttentionMixer", "DenseFeedForward", "ParallelBlock", "SequentialBlock"]
