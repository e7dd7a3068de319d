from .base import (ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, DeferredSum, FixedState, PagedKV, Part, Runtime)
from . import blocks, feedforward, mixers, norms, positions   # noqa: F401  (registers the parts)
from .linear import Linear
from .model import CacheView, DecoderModel, DecoderSpec, EmbeddingTable, LayerCall, LayerSpec

__all__ = ["ARRANGEMENTS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITIONS", "DeferredSum", "FixedState", "PagedKV", "Part",
           "Runtime", "Linear", "CacheView", "DecoderModel", "DecoderSpec", "EmbeddingTable", "LayerCall", "LayerSpec"]
