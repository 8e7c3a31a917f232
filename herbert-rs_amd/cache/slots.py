"""Host-side bookkeeping of slots and pages: plain free lists with strict checks.

A slot stands for one sequence of a running batch; a page holds the keys and
values of PAGE_TOKENS consecutive positions. Nothing here touches the GPU.
The reference keeps one cache object per sequence and drops it with the
sequence (crates/backends/backend_common/src/cpu_backend.rs:182,354-362);
here the storage is allocated once and handed out again.
"""
from ..errors import CacheError

PAGE_TOKENS = 64


class FreeList:
    """Identifiers 0..n-1; each is either free or held, never both, never twice."""

    def __init__(self, count, what):
        if count <= 0:
            raise CacheError(f"a pool of {what}s needs at least one {what}")
        self.count = count
        self.what = what
        self._free = list(range(count - 1, -1, -1))   # pop() hands out the lowest first
        self._held = set()

    def take(self):
        if not self._free:
            raise CacheError(f"no free {self.what} left (all {self.count} are held)")
        ident = self._free.pop()
        self._held.add(ident)
        return ident

    def give_back(self, ident):
        if ident not in self._held:
            raise CacheError(f"{self.what} {ident} is not held (freed twice, or never taken)")
        self._held.remove(ident)
        self._free.append(ident)

    def is_held(self, ident):
        return ident in self._held

    @property
    def free_count(self):
        return len(self._free)

    @property
    def held_count(self):
        return len(self._held)

    def check(self):
        """Every identifier is in exactly one of the two sets."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise CacheError(f"a {self.what} is in the free list twice")
        if free & self._held:
            raise CacheError(f"a {self.what} is both free and held")
        if len(free) + len(self._held) != self.count:
            raise CacheError(f"a {self.what} is lost")


def pages_for(tokens):
    """Pages that `tokens` positions need."""
    return (tokens + PAGE_TOKENS - 1) // PAGE_TOKENS
