"""Parts that layers are put together from; importing the package registers the built-in ones."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward,
                   KVCacheSpec, LayerCache, Mixer, Norm, PAGE, PagedCacheSpec, PagedTensor, Part, PositionEncoding, StateSpec,
                   StepContext)
from .norm import RMSNorm
from .rope import RotaryEmbedding, rope_frequencies
from .attention import PagedAttention
from .mlp import SwiGLU
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
from .model import CachePlan, DecoderModel, ModelSpec, RunEntry, plan_cache

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block", "FeedForward",
    "KVCacheSpec", "LayerCache", "Mixer", "Norm", "PAGE", "PagedCacheSpec", "PagedTensor", "Part", "PositionEncoding", "StateSpec",
    "StepContext", "RMSNorm", "RotaryEmbedding", "rope_frequencies", "PagedAttention", "SwiGLU",
    "PreNormBlock", "LMHead", "TokenEmbedding", "CachePlan", "DecoderModel", "ModelSpec",
    "RunEntry", "plan_cache",
]
