"""One registry from an architecture's name to everything that is particular to it.

An entry holds the configuration class, the builder of the model's
specification, how its checkpoints spell tensor names (weights/names.py) and
how a chat turn is written for it. The name is `architectures[0]` of
config.json, or `model_type` when that is absent; when config.json names
neither, the architecture registered with `default=True` is taken (the
reference selects by `model_type` alone and takes "qwen3" when the key is
missing: crates/core/src/config.rs:95-102,184-185,261-263). An unknown name
is an error that lists the registered ones
(cf. crates/backend_registry/src/lib.rs:235-241).
"""
from dataclasses import dataclass
from typing import Callable, Optional

from ..errors import ConfigError
from .base import read_config_json


@dataclass(frozen=True)
class ChatFormat:
    """How a single user turn (and an optional system prompt) becomes the text that is
    tokenized, and which token ends the model's turn (its id when the tokenizer does not know
    the token). The reference picks the template by model family
    (crates/cli/src/main.rs:260-297) and stops on the end-of-turn token beside eos
    (crates/cli/src/main.rs:616-619)."""
    build_prompt: Callable          # (user text, system text or None) -> str
    end_of_turn: Optional[str] = None
    end_of_turn_id: Optional[int] = None
    # what stands between the token that ends a turn and the next turn's text in a conversation
    # (crates/cli/src/chat.rs:364-381)
    between_turns: str = ""
    # the tokens that open and close a think block, for a cap on its length
    # (crates/cli/src/main.rs:671-684: looked up in the tokenizer, else these ids)
    think_open: Optional[str] = None
    think_close: Optional[str] = None
    think_open_id: Optional[int] = None
    think_close_id: Optional[int] = None
    newline_id: Optional[int] = None


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build_spec: Callable            # config -> ModelSpec
    name_map: object = None         # weights.names.NameMap; None = names as stored
    chat: Optional[ChatFormat] = None


_ARCHITECTURES = {}
_MODEL_TYPES = {}
_DEFAULT = []                       # at most one: the architecture of a config.json that names none


def register_architecture(name, config_class, build_spec, model_types=(), name_map=None, chat=None,
                          default=False):
    """Make `name` (and the given `model_type` strings) resolve to this architecture."""
    arch = Architecture(name, config_class, build_spec, name_map, chat)
    _ARCHITECTURES[name] = arch
    for mt in model_types:
        _MODEL_TYPES[mt] = arch
    if default:
        _DEFAULT[:] = [arch]
    return arch


def registered_architectures():
    return sorted(_ARCHITECTURES)


_plugins_loaded = []


def load_plugins():
    """Import, once, the modules that the environment variable HERBERT_PLUGINS names (separated by
    commas): modules outside this package that register parts or an architecture of their own, so
    that the programs (`bin/trace_run`, `bin/herbert-cli`) and `load` know them as they know the
    library's. The reference's families are compiled in (crates/core/src/config.rs:95-101)."""
    import importlib
    import os
    for name in os.environ.get("HERBERT_PLUGINS", "").split(","):
        name = name.strip()
        if name and name not in _plugins_loaded:
            _plugins_loaded.append(name)
            try:
                importlib.import_module(name)
            except ImportError as e:
                raise ConfigError(f"HERBERT_PLUGINS names {name!r}, which cannot be imported: {e}") from None


def resolve_architecture(raw):
    """The Architecture that a config dict names."""
    load_plugins()
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs:
        name = archs[0]
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(registered_architectures())}")
    model_type = raw.get("model_type")
    if model_type is None:
        if _DEFAULT:
            return _DEFAULT[0]
        raise ConfigError("config.json names neither architectures nor model_type; registered: "
                          + ", ".join(registered_architectures()))
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
