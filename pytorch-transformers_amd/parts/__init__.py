"""Parts that models are put together from: mixers, feed-forwards, norms, position encodings, blocks."""
from .base import Part, StepContext, make_part, register_part, registered_parts
from .linear import Embedding, Linear, OutputHead, QkvTail, TailDone
from .norms import LayerNorm, RMSNorm
from .positions import AlibiPositions, NoPositions, Rotation, RotaryPositions, ScoreBias, alibi_slopes
from .attention import AttentionMixer
from .feedforward import DenseFeedForward, GatedFeedForward, PolyNormFeedForward, RoutedFeedForward, XieluFeedForward
from .blocks import ParallelBlock, PostNormBlock, SandwichBlock, SequentialBlock, ShiftedParallelBlock
from .gated_attention import GatedAttentionMixer
from .linear_attention import DecayLinearAttentionMixer
from .depth import DepthMix, LoopEntry
from .latent_attention import LatentAttentionMixer
from .recurrent import GatedScanMixer, StateSpaceMixer

__all__ = ["Part", "StepContext", "make_part", "register_part", "registered_parts", "Embedding", "Linear",
           "OutputHead", "LayerNorm", "AlibiPositions", "NoPositions", "Rotation", "RotaryPositions", "ScoreBias", "alibi_slopes",
           "AttentionMixer", "DenseFeedForward", "ParallelBlock", "SequentialBlock", "PostNormBlock", "RMSNorm", "DepthMix",
           "LatentAttentionMixer", "GatedScanMixer", "StateSpaceMixer", "GatedFeedForward", "RoutedFeedForward",
           "ShiftedParallelBlock", "GatedAttentionMixer", "DecayLinearAttentionMixer", "SandwichBlock", "LoopEntry",
           "PolyNormFeedForward", "XieluFeedForward"]
