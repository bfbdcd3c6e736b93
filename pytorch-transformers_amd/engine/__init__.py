"""Model assembly, the step function and the generation loop."""
from .spec import (CACHE_FULL, CACHE_STATE, CACHE_WINDOW, CacheGroupSpec, LayerCall, ModelSpec, TensorSpec)

__all__ = ["CACHE_FULL", "CACHE_STATE", "CACHE_WINDOW", "CacheGroupSpec", "LayerCall", "ModelSpec", "TensorSpec"]
