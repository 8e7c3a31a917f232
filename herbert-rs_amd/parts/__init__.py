"""The parts a layer is put together from, and the data that says how."""
from .base import Part, Runtime, StepContext
from .registry import CATEGORIES, build, register, registered
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from . import attention, block, io, mlp, norm, position   # registers the built-in kinds

__all__ = ["CATEGORIES", "LayerSpec", "ModelSpec", "Part", "PartSpec", "Runtime", "ScheduleEntry",
           "StepContext", "build", "register", "registered"]
