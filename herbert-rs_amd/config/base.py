"""Reading config.json and what every architecture's configuration shares.

A configuration class is a frozen dataclass built by `from_dict` from the keys
of the architecture's own config.json. It knows nothing about kernels or
weights; a model builder (see `herbert_rs_amd.models`) turns it into a model
specification.
"""
import json
import os

from ..errors import ConfigError


def read_config_json(path):
    """The dict in `path` (a model folder or the config.json itself)."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path) as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json at {path}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return raw


class Reader:
    """Typed access to a config dict with errors that name the key."""

    def __init__(self, raw):
        self.raw = raw

    def has(self, key):
        return key in self.raw and self.raw[key] is not None

    def integer(self, key, default=None, required=False):
        if not self.has(key):
            if required:
                raise ConfigError(f"config.json: missing {key}")
            return default
        v = self.raw[key]
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                return int(v)
            raise ConfigError(f"config.json: {key} must be an integer, got {v!r}")
        return v

    def number(self, key, default=None, required=False):
        if not self.has(key):
            if required:
                raise ConfigError(f"config.json: missing {key}")
            return default
        v = self.raw[key]
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: {key} must be a number, got {v!r}")
        return float(v)

    def boolean(self, key, default):
        if not self.has(key):
            return default
        v = self.raw[key]
        if not isinstance(v, bool):
            raise ConfigError(f"config.json: {key} must be true or false, got {v!r}")
        return v
