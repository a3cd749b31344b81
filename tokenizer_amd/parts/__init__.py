from .base import (BLOCKS, FEED_FORWARDS, FRAMES, MIXERS, NORMS, POSITIONS, Block, FeedForward, Mixer, Norm, NormFold,
                   Part, PositionEncoding, Registry, Runtime, StoreEpilogue, as_tensor)
from .spec import (CacheNeed, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                   ScheduleEntry, TensorSpec)
from . import norm, position, attention, feed_forward, block  # noqa: F401  (register the built-in parts)
from .model import DecoderModel, LayerCache, build_model, cache_needs, expected_tensors

__all__ = ["BLOCKS", "FEED_FORWARDS", "FRAMES", "MIXERS", "NORMS", "POSITIONS", "Block", "FeedForward", "Mixer", "Norm",
           "NormFold", "Part", "PositionEncoding", "Registry", "Runtime", "StoreEpilogue", "as_tensor", "CacheNeed", "FeedForwardSpec", "LayerSpec",
           "MixerSpec", "ModelSpec", "NormSpec", "PositionSpec", "ScheduleEntry", "TensorSpec",
           "DecoderModel", "LayerCache", "build_model", "cache_needs", "expected_tensors"]
