"""Architectures: each module turns its typed configuration into a ModelSpec and registers itself."""
from . import qwen3

__all__ = ["qwen3"]
