"""What a mixer asks of the cache; a model's layers are grouped by equal needs."""
from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position, or of the last `window` positions only."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """State of a fixed size for each sequence (zero when the sequence starts)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
