"""Typed configurations and the architecture registry."""
from .base import read_config_json
from .registry import (Architecture, ChatFormat, load_config, register_architecture,
                       registered_architectures, resolve_architecture)
from .qwen3 import Qwen3Config

__all__ = ["Architecture", "ChatFormat", "Qwen3Config", "load_config", "read_config_json",
           "register_architecture", "registered_architectures", "resolve_architecture"]
