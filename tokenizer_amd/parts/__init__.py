from .base import (BLOCKS, FEED_FORWARDS, FRAMES, MIXERS, NORMS, POSITIONS, Block, FeedForward, Mixer, Norm, NormFold,
                   Part, PositionEncoding, Registry, Runtime, StoreEpilogue, ScaledSum, SumDelta, as_tensor)
from .spec import (CacheNeed, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                   ScheduleEntry, TensorSpec)
from . import norm, position, attention, feed_forward, block, mlstm, latent, delta, ssm  # noqa: F401  (register the built-in parts)
from .model import DecoderModel, LayerCache, build_model, cache_needs, expected_tensors
from . import streams  # noqa: F401  (the block and the frame over several residual streams)
from . import pair  # noqa: F401  (two mixers side by side)

__all__ = ["BLOCKS", "FEED_FORWARDS", "FRAMES", "MIXERS", "NORMS", "POSITIONS", "Block", "FeedForward", "Mixer", "Norm",
           "NormFold", "Part", "PositionEncoding", "Registry", "Runtime", "StoreEpilogue", "ScaledSum", "SumDelta", "as_tensor", "CacheNeed", "FeedForwardSpec", "LayerSpec",
           "MixerSpec", "ModelSpec", "NormSpec", "PositionSpec", "ScheduleEntry", "TensorSpec",
           "DecoderModel", "LayerCache", "build_model", "cache_needs", "expected_tensors"]
