"""A small MI355X-native model library with generation of its own: one step function over a
paged cache, parts chosen layer by layer, hand-written gfx950 kernels, float32 and bfloat16."""
from . import errors
from .errors import (BackendError, CacheError, ConfigError, HerbertError, ModelLoadError,
                     RequestError)
from . import config, weights, cache, parts, models
from .config import Qwen3Config, load_config, register_architecture
from .engine import Engine, StepEntry

__all__ = ["BackendError", "CacheError", "ConfigError", "Engine", "HerbertError", "ModelLoadError",
           "Qwen3Config", "RequestError", "StepEntry", "load_config", "register_architecture"]
