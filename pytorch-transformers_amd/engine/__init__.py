"""Model assembly, the step function and the generation loop."""
from .spec import (CACHE_CHUNK, CACHE_FULL, CACHE_STATE, CACHE_WINDOW, CacheGroupSpec, LayerCall, ModelSpec, TensorSpec)

__all__ = ["CACHE_CHUNK", "CACHE_FULL", "CACHE_STATE", "CACHE_WINDOW", "CacheGroupSpec", "LayerCall", "ModelSpec", "TensorSpec"]
