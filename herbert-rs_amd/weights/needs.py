"""What a model asks of its weight files: names, shapes, and how to draw a random stand-in."""
from dataclasses import dataclass
from typing import Callable, Optional, Tuple


@dataclass(frozen=True)
class TensorNeed:
    """One tensor that a part reads by name.

    role says what the tensor is and thereby how the random-weights mode draws it when `init`
    is not given: "matrix" (a linear layer's [out, in]) and "table" (the embedding) are
    N(0, std), "scale" (a norm's weight) is 1 + N(0, norm_std), "index" (an integer table) is
    zeros. A part whose tensor is none of these (a bias, a convolution's taps, a decay rate)
    brings its own `init(shape, generator, device, std, norm_std) -> float32 or int32 tensor`;
    nothing else in the library has to know the new kind.
    """
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: Optional[Callable] = None
