"""The hand-written gfx950 kernels and their host-side checks."""
from . import build, lib, ops

__all__ = ["build", "lib", "ops"]
