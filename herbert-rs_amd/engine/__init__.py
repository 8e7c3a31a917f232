"""Model, step function, generation loop and trace replay."""
from .batch import BatchMeta, StepEntry
from .engine import Engine
from .generate import GenerationResult, Generator
from .model import Model

__all__ = ["BatchMeta", "Engine", "GenerationResult", "Generator", "Model", "StepEntry"]
