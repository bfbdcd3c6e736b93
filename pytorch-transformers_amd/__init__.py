"""A small MI355X-native model library with generation: configuration, weights, parts, cache,
step function, generation loop and sampling for the Falcon architecture, on hand-written gfx950
HIP kernels.  Import name: ``pytorch_transformers_amd``."""
from .config import AutoConfig, ConfigError, FalconConfig, GenerationConfig, register
from .engine import falcon as _falcon  # registers model_type "falcon"  # noqa: F401
from .auto import AutoModelForCausalLM
from .pipeline import TextGenerationPipeline, pipeline
from .sampling.custom import LogitsProcessor, LogitsProcessorList, StoppingCriteria, StoppingCriteriaList
from .streaming import BaseStreamer, TextIteratorStreamer, TextStreamer

__version__ = "0.1.0"
__all__ = ["AutoConfig", "AutoModelForCausalLM", "BaseStreamer", "ConfigError", "FalconConfig", "GenerationConfig",
           "LogitsProcessor", "LogitsProcessorList", "StoppingCriteria", "StoppingCriteriaList", "TextGenerationPipeline",
           "TextIteratorStreamer", "TextStreamer", "pipeline", "register"]
