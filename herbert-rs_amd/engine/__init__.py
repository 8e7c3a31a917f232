"""Model, step function, generation loop and trace replay."""
from .batch import BatchMeta, StepEntry
from .engine import Engine
from .model import Model

__all__ = ["BatchMeta", "Engine", "Model", "StepEntry"]
