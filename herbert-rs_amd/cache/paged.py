"""The cache on the GPU: paged keys and values per group of layers, and fixed-size state.

Layers (more exactly: the entries of a model's schedule that own a cache) with
the same need share a group. A group of keys and values owns one pool
[entries, 2, pages, kv_heads, PAGE_TOKENS, head_dim], a page list of its own
and a page table [slots, pages per slot]; the page index is shared by the
group's entries, so one table serves them all. A group with a window gives
back the pages that no later query can see. A group of fixed-size state owns
[entries, slots, *shape] and is cleared for a slot when the slot is taken.

Beyond the slots and pages that sequences can hold there is one more of each:
the padding slot (`Cache.pad_slot`), whose page table points at the padding page
everywhere. Rows that fill a step up to a fixed size (a decode step that is
replayed as a graph of the next larger batch size) write and read there and
nowhere else; no sequence ever holds either.

Per slot the host keeps the length (positions held = next position), as the
reference keeps `seq_len` beside its storage
(crates/backends/backend_common/src/kv_cache.rs:270-273).
"""
from dataclasses import dataclass

import numpy as np
import torch

from ..errors import CacheError
from .needs import KVNeed, StateNeed
from .slots import PAGE_TOKENS, FreeList, pages_for


@dataclass
class LayerKV:
    """What an attention kernel needs of one schedule entry's cache."""
    k: torch.Tensor            # [pages, kv_heads, PAGE_TOKENS, head_dim]
    v: torch.Tensor            # [pages, kv_heads, head_dim, PAGE_TOKENS]: tokens contiguous
    page_table: torch.Tensor   # int32 [slots, pages per slot]
    page_size: int
    window: int                # 0 = all keys


class KVGroup:
    def __init__(self, need, entries, n_pages, n_slots, max_positions, dtype, device):
        self.need = need
        self.entries = list(entries)
        self.pages = FreeList(n_pages, "page")
        self.pages_per_slot = pages_for(max_positions)
        # (one page and one slot more than sequences can hold: the padding page and the padding slot)
        self.pool = torch.zeros((len(self.entries), 2, n_pages + 1, need.kv_heads, PAGE_TOKENS,
                                 need.head_dim), dtype=dtype, device=device)
        self.table_host = np.full((n_slots, self.pages_per_slot), -1, dtype=np.int32)
        # entries of the device table that are not held point at page 0: a kernel never reads
        # them for a valid position, and an index that is always in range cannot fault
        self.table = torch.zeros((n_slots + 1, self.pages_per_slot), dtype=torch.int32, device=device)
        self.table[n_slots] = n_pages
        # a slot holds the logical pages [first_page, held_end): it fills from the front as it grows,
        # a window gives pages back at the front, a roll-back at the end
        self.first_page = np.zeros(n_slots, dtype=np.int64)
        self.held_end = [0] * n_slots

    def view(self, entry):
        i = self.entries.index(entry)
        n_pages = self.pool.shape[2]         # (with the padding page)
        k = self.pool[i, 0]
        v = self.pool[i, 1].view(n_pages, self.need.kv_heads, self.need.head_dim, PAGE_TOKENS)
        return LayerKV(k, v, self.table, PAGE_TOKENS, int(self.need.window or 0))

    def pages_missing(self, slot, new_length):
        """How many pages `ensure(slot, new_length)` would take."""
        return max(0, pages_for(new_length) - max(self.held_end[slot], int(self.first_page[slot])))

    def ensure(self, slot, new_length):
        """Hold a page for every position below new_length that a query may still see."""
        last = pages_for(new_length)
        first_new = max(self.held_end[slot], int(self.first_page[slot]))
        if first_new >= last:
            return
        row = self.table_host[slot]
        for p in range(first_new, last):
            row[p] = self.pages.take()
        self.held_end[slot] = last
        self._upload(slot, first_new, last)

    def _upload(self, slot, a, b):
        self.table[slot, a:b] = torch.from_numpy(np.maximum(self.table_host[slot, a:b], 0)).to(
            self.table.device)

    def release_unseen(self, slot, length):
        """With a window: give back pages wholly before the oldest key a later query sees."""
        if not self.need.window:
            return
        # a query at position >= length sees keys >= length + 1 - window
        oldest = length + 1 - self.need.window
        row = self.table_host[slot]
        p = int(self.first_page[slot])
        while (p + 1) * PAGE_TOKENS <= oldest:
            if row[p] >= 0:
                self.pages.give_back(int(row[p]))
                row[p] = -1
            p += 1
        self.first_page[slot] = p

    def can_truncate(self, slot, length):
        if self.need.window:
            oldest = max(0, length + 1 - self.need.window)   # oldest key the next query sees
            if self.first_page[slot] * PAGE_TOKENS > oldest:
                return False
        return True

    def truncate(self, slot, length):
        """Give back the pages wholly behind `length`. What the kept last page holds behind
        `length` stays where it is: no query sees it (keys are counted, not marked) and the next
        tokens overwrite it."""
        row = self.table_host[slot]
        if not self.can_truncate(slot, length):
            raise CacheError("cannot roll a windowed cache back past keys it has given up")
        for p in range(pages_for(length), self.held_end[slot]):
            if row[p] >= 0:
                self.pages.give_back(int(row[p]))
                row[p] = -1
        self.held_end[slot] = min(self.held_end[slot], pages_for(length))

    def free_slot(self, slot):
        row = self.table_host[slot]
        for p in np.nonzero(row >= 0)[0]:
            self.pages.give_back(int(row[p]))
        row[:] = -1
        self.first_page[slot] = 0
        self.held_end[slot] = 0


class StateGroup:
    def __init__(self, need, entries, n_slots, device):
        self.need = need
        self.entries = list(entries)
        self.data = torch.zeros((len(self.entries), n_slots + 1) + tuple(need.shape), dtype=need.dtype,
                                device=device)      # (the last: the padding slot's)

    def view(self, entry):
        return self.data[self.entries.index(entry)]

    def clear_slot(self, slot):
        self.data[:, slot].zero_()


class Cache:
    """Slots, their lengths, and the groups of storage behind them.

    `needs` maps a schedule entry (an int) to its need (KVNeed, StateNeed, or a
    tuple of them); entries that read another entry's cache are not in it.
    `max_tokens` is the most tokens that live sequences hold at any time, each
    sequence's count rounded up to a multiple of PAGE_TOKENS.
    """

    def __init__(self, needs, max_tokens, max_positions, dtype, device, max_slots=None):
        n_pages = pages_for(max(int(max_tokens), 1))
        self.n_pages = n_pages
        self.n_slots = int(max_slots) if max_slots else n_pages
        self.max_positions = int(max_positions)
        self.pad_slot = self.n_slots        # never handed out: where a step's padding rows write and read
        self.slots = FreeList(self.n_slots, "slot")
        self.lengths = np.zeros(self.n_slots, dtype=np.int64)
        self.kv_groups = {}
        self.state_groups = {}
        self._kv_of = {}
        self._state_of = {}
        by_need = {}
        for entry, need in needs.items():
            for one in (need if isinstance(need, (tuple, list)) else (need,)):
                by_need.setdefault(one, []).append(entry)
        for need, entries in by_need.items():
            if isinstance(need, KVNeed):
                group = KVGroup(need, entries, n_pages, self.n_slots, max_positions, dtype, device)
                self.kv_groups[need] = group
                for e in entries:
                    self._kv_of[e] = group
            elif isinstance(need, StateNeed):
                group = StateGroup(need, entries, self.n_slots, device)
                self.state_groups[need] = group
                for e in entries:
                    self._state_of.setdefault(e, []).append(group)
            else:
                raise CacheError(f"unknown cache need {need!r}")

    @staticmethod
    def bytes_needed(needs, max_tokens, dtype, max_slots=None):
        """The GPU memory that a cache of these needs takes: the pools of keys and values (by
        pages) and the fixed-size state (by slots), as the constructor allocates them."""
        n_pages = pages_for(max(int(max_tokens), 1))
        n_slots = (int(max_slots) if max_slots else n_pages) + 1        # with the padding slot
        n_pages += 1                                                     # and the padding page
        element = torch.empty((), dtype=dtype).element_size()
        by_need = {}
        for entry, need in needs.items():
            for one in (need if isinstance(need, (tuple, list)) else (need,)):
                by_need[one] = by_need.get(one, 0) + 1
        total = 0
        for need, entries in by_need.items():
            if isinstance(need, KVNeed):
                total += entries * 2 * n_pages * PAGE_TOKENS * need.kv_heads * need.head_dim * element
            elif isinstance(need, StateNeed):
                per_slot = 1
                for d in need.shape:
                    per_slot *= int(d)
                total += entries * n_slots * per_slot * torch.empty((), dtype=need.dtype).element_size()
        return total

    # ---- slots
    def alloc_slot(self):
        slot = self.slots.take()
        self.lengths[slot] = 0
        for g in self.state_groups.values():
            g.clear_slot(slot)
        return slot

    def free_slot(self, slot):
        self.slots.give_back(slot)
        for g in self.kv_groups.values():
            g.free_slot(slot)
        self.lengths[slot] = 0

    def length(self, slot):
        if not self.slots.is_held(slot):
            raise CacheError(f"slot {slot} is not held")
        return int(self.lengths[slot])

    # ---- one step
    def reserve(self, slot, new_tokens):
        """Make room for `new_tokens` more positions of a slot (before the step runs)."""
        new_length = self.length(slot) + int(new_tokens)
        if new_length > self.max_positions:
            raise CacheError(f"slot {slot}: {new_length} positions exceed the model's "
                             f"{self.max_positions}")
        for g in self.kv_groups.values():
            g.ensure(slot, new_length)
        return new_length

    def reserve_all(self, wanted):
        """`reserve` for every (slot, new tokens) of a step, all or nothing: the pages that each
        group needs are counted first, and a step that does not fit raises CacheError with the
        cache unchanged."""
        targets = []
        for slot, new_tokens in wanted:
            new_length = self.length(slot) + int(new_tokens)
            if new_length > self.max_positions:
                raise CacheError(f"slot {slot}: {new_length} positions exceed the model's "
                                 f"{self.max_positions}")
            targets.append((slot, new_length))
        for g in self.kv_groups.values():
            need = sum(g.pages_missing(slot, n) for slot, n in targets)
            if need > g.pages.free_count:
                raise CacheError(f"the step needs {need} more pages of {PAGE_TOKENS} tokens but only "
                                 f"{g.pages.free_count} of {g.pages.count} are free")
        for slot, new_length in targets:
            for g in self.kv_groups.values():
                g.ensure(slot, new_length)

    def save_state(self, slots):
        """A copy of the fixed-size state of `slots` (None for a cache that has none): what
        `restore_state` puts back when the step that was to change it has failed."""
        if not self.state_groups:
            return None
        index = torch.tensor(sorted(set(int(s) for s in slots)), dtype=torch.long)
        saved = []
        for g in self.state_groups.values():
            at = index.to(g.data.device)
            saved.append((g, at, g.data.index_select(1, at)))
        return saved

    def restore_state(self, saved):
        for g, at, data in saved or ():
            g.data.index_copy_(1, at, data)

    def unreserve(self, slot):
        """Give back what was reserved for a step that did not run: the pages behind the slot's
        committed length."""
        length = self.length(slot)
        for g in self.kv_groups.values():
            g.truncate(slot, length)

    def commit(self, slot, new_tokens):
        """The step has run: the slot is longer; windowed groups give up what is out of sight."""
        self.lengths[slot] += int(new_tokens)
        for g in self.kv_groups.values():
            g.release_unseen(slot, int(self.lengths[slot]))

    @property
    def rolls_back_freely(self):
        """True where `truncate` never refuses a length within the slot's own: no per-sequence
        state, no group that gives keys up as a sequence grows."""
        return not self.state_groups and all(not g.need.window for g in self.kv_groups.values())

    def truncate(self, slot, length):
        """Roll a slot back to its first `length` positions (the reference's truncate_kv,
        crates/backends/backend_common/src/cpu_backend.rs:527-543). Fixed-size state cannot be
        rolled back and refuses."""
        if length > self.length(slot) or length < 0:
            raise CacheError(f"cannot truncate slot {slot} of length {self.length(slot)} to {length}")
        if self.state_groups and length != self.length(slot):
            raise CacheError("a cache with per-sequence state cannot be rolled back")
        for g in self.kv_groups.values():       # refuse before anything is given back
            if not g.can_truncate(slot, length):
                raise CacheError("cannot roll a windowed cache back past keys it has given up")
        for g in self.kv_groups.values():
            g.truncate(slot, length)
        self.lengths[slot] = length

    # ---- views for the parts
    def kv_view(self, entry):
        return self._kv_of[entry].view(entry)

    def state_views(self, entry):
        return [g.view(entry) for g in self._state_of.get(entry, [])]

    def check(self):
        """Bookkeeping invariants: nothing lost, nothing held twice."""
        self.slots.check()
        for g in self.kv_groups.values():
            g.pages.check()
            held = g.table_host[g.table_host >= 0]
            if len(set(held.tolist())) != len(held):
                raise CacheError("a page is in two places of the page table")
            if len(held) != g.pages.held_count:
                raise CacheError("held pages and the page table disagree")
            for slot in range(self.n_slots):
                if not self.slots.is_held(slot) and (g.table_host[slot] >= 0).any():
                    raise CacheError(f"free slot {slot} still holds pages")
                has = np.nonzero(g.table_host[slot] >= 0)[0].tolist()
                first, end = int(g.first_page[slot]), g.held_end[slot]
                if has != list(range(first, end)):
                    raise CacheError(f"slot {slot} holds the pages {has}, not the stretch [{first}, {end}) "
                                     "it keeps count of")
