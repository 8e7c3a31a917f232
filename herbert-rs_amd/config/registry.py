"""One registry from an architecture's name to its configuration class and model builder.

The name is `architectures[0]` of config.json, or `model_type` when that is
absent (the reference selects by `model_type` alone and takes "qwen3" when
the key is missing: crates/core/src/config.rs:95-102,184-185,261-263).
An unknown name is an error that lists the registered ones
(cf. crates/backend_registry/src/lib.rs:235-241).
"""
from dataclasses import dataclass
from typing import Callable

from ..errors import ConfigError
from .base import read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build_spec: Callable      # config -> ModelSpec


_ARCHITECTURES = {}
_MODEL_TYPES = {}
DEFAULT_MODEL_TYPE = "qwen3"


def register_architecture(name, config_class, build_spec, model_types=()):
    """Make `name` (and the given `model_type` strings) resolve to this architecture."""
    arch = Architecture(name, config_class, build_spec)
    _ARCHITECTURES[name] = arch
    for mt in model_types:
        _MODEL_TYPES[mt] = arch
    return arch


def registered_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(raw):
    """The Architecture that a config dict names."""
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs:
        name = archs[0]
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(registered_architectures())}")
    model_type = raw.get("model_type", DEFAULT_MODEL_TYPE)
    if model_type in _MODEL_TYPES:
        return _MODEL_TYPES[model_type]
    raise ConfigError(
        f"unknown model_type {model_type!r}; registered: {', '.join(sorted(_MODEL_TYPES))} "
        f"(architectures: {', '.join(registered_architectures())})")


def load_config(path):
    """(Architecture, typed configuration) of a model folder or a config.json."""
    raw = read_config_json(path)
    arch = resolve_architecture(raw)
    return arch, arch.config_class.from_dict(raw)
