from .base import (ARRANGEMENTS, CONNECTORS, FEED_FORWARDS, FILTERS, MIXERS, NORMS, POSITIONS, DeferredSum, FixedState, PagedKV, Part, Runtime)
from . import blocks, connectors, feedforward, filters, gates, mixers, norms, positions, recurrent, token_inputs   # noqa: F401  (registers the parts)
from .linear import Linear
from .model import CacheView, DecoderModel, DecoderSpec, EmbeddingTable, LayerCall, LayerSpec

__all__ = ["ARRANGEMENTS", "CONNECTORS", "FEED_FORWARDS", "FILTERS", "MIXERS", "NORMS", "POSITIONS", "DeferredSum", "FixedState", "PagedKV", "Part",
           "Runtime", "Linear", "CacheView", "DecoderModel", "DecoderSpec", "EmbeddingTable", "LayerCall", "LayerSpec"]
