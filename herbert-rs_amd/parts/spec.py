"""The data that describes a model: parts chosen layer by layer, and the order they run in.

An architecture's builder (see `herbert_rs_amd.models`) turns a typed
configuration into a ModelSpec; nothing below this level knows which model it
is in. A part is named by its kind (a key of the registry of its category) and
takes every size and constant as a parameter.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: how its parts are arranged (`block`) and which parts they are."""
    block: PartSpec            # the arrangement, e.g. "prenorm"
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Dict[str, PartSpec]  # by the role the block gives them, e.g. "input", "post_mixer"


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer. `cache` None: the entry owns a cache of its own; an int: it reads
    the cache of that earlier entry of the schedule and writes none."""
    layer: int
    cache: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    head: PartSpec
    eos_token_id: Optional[int] = None
