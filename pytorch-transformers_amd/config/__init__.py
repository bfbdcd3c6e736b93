"""Typed configurations, the architecture registry and generation options."""
from .base import CONFIG_NAME, ConfigError, ModelConfig
from .falcon import FalconConfig
from .generation import GENERATION_CONFIG_NAME, GenerationConfig
from .registry import AutoConfig, known_model_types, lookup, register, unregister

__all__ = ["CONFIG_NAME", "ConfigError", "ModelConfig", "FalconConfig", "GENERATION_CONFIG_NAME", "GenerationConfig",
           "AutoConfig", "known_model_types", "lookup", "register", "unregister"]
