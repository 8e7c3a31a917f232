"""A small MI355X-native model library with generation of its own: one step function over a
paged cache, parts chosen layer by layer, hand-written gfx950 kernels, float32 and bfloat16."""
from . import errors
from .errors import (BackendError, CacheError, ConfigError, HerbertError, ModelLoadError,
                     RequestError)
from . import config, weights, cache, parts, models
from .config import Qwen3Config, load_config, register_architecture
from .engine import Engine, StepEntry
from .sampling import SamplingParams
from .api import generate, load, write_random_model

__all__ = ["BackendError", "CacheError", "ConfigError", "Engine", "HerbertError", "ModelLoadError",
           "Qwen3Config", "RequestError", "SamplingParams", "StepEntry", "generate", "load", "load_config",
           "register_architecture", "write_random_model"]
