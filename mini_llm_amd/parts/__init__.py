from .attention import CausalSelfAttention, NormedHeadAttention
from .base import (
    BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS,
    Block, FeedForward, KVNeed, LayerContext, Mixer, Norm, Part, PositionEncoding, StateNeed,
    make_part, register_part,
)
from .block import BranchNormBlock, ParallelBlock, PostNormBlock, PreNormBlock, SandwichNormBlock
from .differential_attention import DifferentialAttention
from .embedding import LinearHead, TiedHead, TokenEmbedding
from .feedforward import ClampedGatedMLP, DenseMLP, GatedMLP
from .latent_attention import LatentAttention
from .linear import Linear
from .norms import LayerNorm, RMSNorm
from .positions import LearnedPositions, RotaryEncoding
from .projection_attention import ProjectionNormAttention
from .rotary_attention import RotaryAttention
from .routed import RoutedExperts
from .recurrent import DecayedLinearAttention, MatrixMemoryMixer, ParallelMixer

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS",
    "Block", "FeedForward", "KVNeed", "LayerContext", "Mixer", "Norm", "Part", "PositionEncoding", "StateNeed",
    "make_part", "register_part",
    "CausalSelfAttention", "PreNormBlock", "TiedHead", "TokenEmbedding", "DenseMLP", "Linear", "LayerNorm", "LearnedPositions",
    "NormedHeadAttention", "LatentAttention", "BranchNormBlock", "ProjectionNormAttention", "DecayedLinearAttention",
    "MatrixMemoryMixer", "ParallelMixer", "PostNormBlock", "SandwichNormBlock", "DifferentialAttention", "LinearHead", "GatedMLP", "RMSNorm", "RotaryEncoding", "ClampedGatedMLP", "ParallelBlock", "RotaryAttention", "RoutedExperts",
]
