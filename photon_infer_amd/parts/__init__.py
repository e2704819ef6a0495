"""Parts that layers are put together from; importing the package registers the built-in ones."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward,
                   KVCacheSpec, LayerCache, Mixer, Norm, PAGE, PagedCacheSpec, PagedTensor, Part, PositionEncoding, StateSpec,
                   StepContext)
from .norm import LayerNorm, RMSNorm
from .rope import RotaryEmbedding, rope_frequencies
from .attention import PagedAttention
from .sink_attention import SinkWindowAttention
from .latent_attention import LatentAttention
from .matrix_memory import MatrixMemory
from .state_space import StateSpaceMixer
from .delta_rule import ChannelDeltaRule, GatedDeltaRule
from .diff_attention import DifferentialAttention
from .linear_attention import GatedLinearAttention
from .mlp import ClampedGLU, SquaredReluMLP, SwiGLU
from .routed_experts import RoutedExperts
from .block import OutputNormBlock, PreNormBlock, SandwichBlock, SideBySide
from .embedding import LMHead, PositionedEmbedding, TokenEmbedding
from .model import CachePlan, DecoderModel, ModelSpec, RunEntry, plan_cache

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block", "FeedForward",
    "KVCacheSpec", "LayerCache", "Mixer", "Norm", "PAGE", "PagedCacheSpec", "PagedTensor", "Part", "PositionEncoding", "StateSpec",
    "StepContext", "RMSNorm", "RotaryEmbedding", "rope_frequencies", "PagedAttention", "SwiGLU",
    "PreNormBlock", "OutputNormBlock", "SinkWindowAttention", "MatrixMemory", "RoutedExperts", "LMHead", "TokenEmbedding", "CachePlan", "DecoderModel", "ModelSpec",
    "RunEntry", "plan_cache", "StateSpaceMixer", "ChannelDeltaRule", "ClampedGLU", "SideBySide", "PositionedEmbedding", "LatentAttention",
    "LayerNorm", "GatedDeltaRule", "DifferentialAttention", "GatedLinearAttention", "SquaredReluMLP", "SandwichBlock",
]
