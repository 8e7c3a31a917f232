"""What a model asks of its weight files: names, shapes and roles."""
from dataclasses import dataclass
from typing import Tuple


@dataclass(frozen=True)
class TensorNeed:
    """One tensor that a part reads by name.

    role: "matrix" (a linear layer's [out, in]), "table" (the embedding),
    "scale" (a norm's weight, near one), "index" (an integer table).
    """
    shape: Tuple[int, ...]
    role: str = "matrix"
