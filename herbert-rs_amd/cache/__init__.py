"""Slots, paged keys and values per group of layers, fixed-size per-sequence state."""
from .needs import KVNeed, StateNeed
from .paged import Cache, KVGroup, LayerKV, StateGroup
from .slots import PAGE_TOKENS, FreeList, pages_for

__all__ = ["Cache", "FreeList", "KVGroup", "KVNeed", "LayerKV", "PAGE_TOKENS", "StateGroup",
           "StateNeed", "pages_for"]
