"""Host-side bookkeeping of the cache: sequence slots and pages.

The reference keeps one `PageAllocator` (a LIFO free list over one VRAM pool with
range and double-free asserts, crates/braidinfer-runtime/src/paged_kv.rs:83-181) and a
single `SequenceState` for the whole model (model/mod.rs:88).  Here there is a slot per
sequence of a batch, and misuse is an error the caller can catch, not an assert.
"""
from __future__ import annotations

from typing import List

from ..errors import CacheError


class PagePool:
    """`n_pages` page indices; `alloc(n)` takes n or none (atomic), `free` gives back."""

    def __init__(self, n_pages: int):
        if n_pages <= 0:
            raise CacheError(f"a page pool needs at least one page, got {n_pages}")
        self.n_pages = n_pages
        self._free: List[int] = list(range(n_pages - 1, -1, -1))   # LIFO: page 0 first
        self._held = [False] * n_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def held_count(self) -> int:
        return self.n_pages - len(self._free)

    def alloc(self, n: int) -> List[int]:
        if n < 0:
            raise CacheError(f"cannot allocate {n} pages")
        if n > len(self._free):
            raise CacheError(f"out of cache pages: {n} wanted, {len(self._free)} of {self.n_pages} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def free(self, pages) -> None:
        pages = list(pages)
        for p in pages:
            if not 0 <= p < self.n_pages:
                raise CacheError(f"page {p} is outside the pool of {self.n_pages}")
            if not self._held[p]:
                raise CacheError(f"page {p} freed twice (or never allocated)")
        if len(set(pages)) != len(pages):
            raise CacheError("a page appears twice in one free")
        for p in pages:
            self._held[p] = False
            self._free.append(p)


class SlotAllocator:
    """Slots 0..n-1, one per live sequence."""

    def __init__(self, n_slots: int):
        if n_slots <= 0:
            raise CacheError(f"need at least one slot, got {n_slots}")
        self.n_slots = n_slots
        self._free: List[int] = list(range(n_slots - 1, -1, -1))
        self._live = [False] * n_slots

    @property
    def free_count(self) -> int:
        return len(self._free)

    def live_slots(self) -> List[int]:
        return [i for i, l in enumerate(self._live) if l]

    def alloc(self) -> int:
        if not self._free:
            raise CacheError(f"out of sequence slots: all {self.n_slots} are live")
        s = self._free.pop()
        self._live[s] = True
        return s

    def check_live(self, slot: int) -> None:
        if not isinstance(slot, int) or not 0 <= slot < self.n_slots:
            raise CacheError(f"slot {slot!r} is outside 0..{self.n_slots - 1}")
        if not self._live[slot]:
            raise CacheError(f"slot {slot} is not live (freed or never allocated)")

    def free(self, slot: int) -> None:
        if not isinstance(slot, int) or not 0 <= slot < self.n_slots:
            raise CacheError(f"slot {slot!r} is outside 0..{self.n_slots - 1}")
        if not self._live[slot]:
            raise CacheError(f"slot {slot} freed twice (or never allocated)")
        self._live[slot] = False
        self._free.append(slot)
