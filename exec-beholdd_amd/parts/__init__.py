"""Parts that models are put together from; see base.py for the interfaces."""

from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheNeed, LayerCache,
                   Registry, StepContext)
from .linear import Linear
from .norm import RMSNorm
from .rope import NoPositionEncoding, RotaryEncoding
from .attention import GQAAttention
from .mlp import SwiGLU
from .block import PreNormBlock
from .embedding import Embedding, LMHead

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "CacheNeed", "LayerCache",
           "Registry", "StepContext", "Linear", "RMSNorm", "NoPositionEncoding", "RotaryEncoding",
           "GQAAttention", "SwiGLU", "PreNormBlock", "Embedding", "LMHead"]
