"""The cache of a model: a slot per sequence, paged keys and values per layer group,
and a fixed-size state area per sequence.

Layout (decided for the attention kernels of this library, not taken from the
reference, whose page holds all layers of 64 tokens as f32,
crates/braidinfer-runtime/src/paged_kv.rs:17-21): a *group* gathers the cache units
whose needs are equal (kv heads, widths of what is kept per token, full or windowed).  A
group owns one page pool and one block table `[slot, page index in sequence] -> page`;
every unit of the group owns storage `[n_pages, elements of a page]` indexed by the same
page numbers.  A page holds, for its 64 tokens, first the keys of every kv head
(`[kv_heads, 64 * key_dim]`), then the values (`[kv_heads, 64 * value_dim]`); the two widths
may differ and the second may be zero (a mixer that keeps one row per token).  What lies
inside a head's block is the mixer's business: the attention part of this library keeps
keys as `[token, head_dim]` after rotation and values transposed as `[head_dim, token]`
(the operand layout of the matrix-core attention kernels).  A windowed group returns pages
that lie wholly before the window to its pool after every step.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from ..errors import CacheError
from .allocator import PagePool, SlotAllocator

PAGE_TOKENS = 64


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer asks of the cache for one unit: rows that grow with the sequence.
    Per token and kv head it keeps `head_dim` elements of keys and `value_dim` elements of
    values (None: as many as of keys; 0: none)."""

    kv_heads: int
    head_dim: int
    window: Optional[int] = None      # None: all keys; W: the last W positions
    value_dim: Optional[int] = None
    # Which rows later tokens can still see, for mixers with another rule than "all" or "the last W": a
    # function from a sequence's length to the first position that stays visible (rows before it are never
    # read again, pages wholly before it go back to the pool).  None: the window's rule.  Units whose needs
    # are to share a group name the same function object.
    live_from: Optional[Callable[[int], int]] = None

    @property
    def key_dim(self) -> int:
        return self.head_dim

    def first_live(self, length: int) -> int:
        """The first position of a sequence of `length` tokens that a later token may still read."""
        if self.live_from is not None:
            return max(0, min(int(length), int(self.live_from(int(length)))))
        return 0 if self.window is None else max(0, length - self.window + 1)

    @property
    def val_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size per-sequence state of a mixer (zeroed when a slot is allocated)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class _PinnedStaging:
    """Pinned host memory for the changed pieces of a block table on their way to the device: two
    halves used in turn; a half is written again only when every copy made from it has finished
    (an event recorded when the half was left).  Copies from it need not wait for the device, so a
    step that takes a new page does not hold the host up."""

    def __init__(self, half: int):
        self.half = half
        self.buf = torch.empty(2 * half, dtype=torch.int32, pin_memory=True)
        self.turn = 0
        self.used = 0
        self.left = [None, None]        # per half: the event behind the last copy made from it

    def take(self, n: int) -> Optional[torch.Tensor]:
        """`n` integers of staging memory, or None when a piece is larger than a half."""
        if n > self.half:
            return None
        if self.used + n > self.half:
            ev = self.left[self.turn] or torch.cuda.Event()
            ev.record()
            self.left[self.turn] = ev
            self.turn ^= 1
            self.used = 0
            if self.left[self.turn] is not None:
                self.left[self.turn].synchronize()
        o = self.turn * self.half + self.used
        self.used += n
        return self.buf[o:o + n]


class CacheGroup:
    def __init__(self, need: CacheNeed, unit_ids: Sequence[int], n_pages: int, n_slots: int,
                 max_pages_per_seq: int, page_tokens: int, dtype: torch.dtype, device):
        self.need = need
        self.unit_ids = list(unit_ids)
        self.page_tokens = page_tokens
        self.pool = PagePool(n_pages)
        self.max_pages_per_seq = max_pages_per_seq
        self.pages: List[List[int]] = [[] for _ in range(n_slots)]   # by page index in sequence; -1 = returned
        self.first_page: List[int] = [0] * n_slots                    # pages before this index were returned
        self.device = torch.device(device)
        self.table_cpu = torch.full((n_slots, max_pages_per_seq), -1, dtype=torch.int32)
        self.table_dev = self.table_cpu.to(self.device) if self.device.type != "cpu" else self.table_cpu
        self._dirty: Dict[int, Tuple[int, int]] = {}
        self._staging = _PinnedStaging(max(4096, 2 * max_pages_per_seq)) if self.device.type == "cuda" else None
        if need.kv_heads <= 0 or need.key_dim <= 0 or need.val_dim < 0:
            raise CacheError(f"a cache unit needs kv heads and a key width above zero, got {need}")
        self.key_elems = need.kv_heads * page_tokens * need.key_dim        # of one page
        self.page_elems = self.key_elems + need.kv_heads * page_tokens * need.val_dim
        self.storage: Dict[int, torch.Tensor] = {}
        if dtype is not None:
            for u in self.unit_ids:
                self.storage[u] = torch.zeros((n_pages, self.page_elems), dtype=dtype, device=self.device)

    # -- views of a unit's storage ----------------------------------------------------------
    def keys(self, unit: int) -> torch.Tensor:
        """[pages, kv_heads, page_tokens * key_dim]: every head's block of keys, page by page."""
        return self.storage[unit][:, :self.key_elems].view(-1, self.need.kv_heads, self.page_tokens * self.need.key_dim)

    def values(self, unit: int) -> torch.Tensor:
        """[pages, kv_heads, page_tokens * value_dim]."""
        return self.storage[unit][:, self.key_elems:].view(-1, self.need.kv_heads, self.page_tokens * self.need.val_dim)

    def storage_view(self, unit: int) -> torch.Tensor:
        """Keys and values of equal width as one tensor [pages, 2, kv_heads, page_tokens, head_dim]
        (what this library's attention kernels take); the flat [pages, page elements] otherwise."""
        n = self.need
        if n.val_dim == n.key_dim:
            return self.storage[unit].view(-1, 2, n.kv_heads, self.page_tokens, n.key_dim)
        return self.storage[unit]

    # -- bookkeeping, all on the host ------------------------------------------------
    def pages_needed(self, slot: int, new_len: int) -> int:
        return max(0, -(-new_len // self.page_tokens) - len(self.pages[slot]))

    def grow(self, slot: int, new_len: int) -> None:
        have = len(self.pages[slot])
        want = -(-new_len // self.page_tokens)
        if want > self.max_pages_per_seq:
            raise CacheError(f"sequence of {new_len} tokens exceeds the cache's longest sequence "
                             f"({self.max_pages_per_seq * self.page_tokens})")
        if want > have:
            new = self.pool.alloc(want - have)
            self.pages[slot].extend(new)
            self.table_cpu[slot, have:want] = torch.tensor(new, dtype=torch.int32)
            self._mark(slot, have, want)

    def trim(self, slot: int, length: int) -> None:
        """Return pages that no later query can see (by the window, or by the need's own rule)."""
        if self.need.window is None and self.need.live_from is None:
            return
        first_live = self.need.first_live(length) // self.page_tokens
        lo = self.first_page[slot]
        if first_live > lo:
            dead = [p for p in self.pages[slot][lo:first_live] if p >= 0]
            self.pool.free(dead)
            for i in range(lo, first_live):
                self.pages[slot][i] = -1
            self.table_cpu[slot, lo:first_live] = -1
            self._mark(slot, lo, first_live)
            self.first_page[slot] = first_live

    def release(self, slot: int) -> None:
        self.pool.free([p for p in self.pages[slot] if p >= 0])
        n = len(self.pages[slot])
        if n:
            self.table_cpu[slot, :n] = -1
            self._mark(slot, 0, n)
        self.pages[slot] = []
        self.first_page[slot] = 0

    def _mark(self, slot, lo, hi):
        if slot in self._dirty:
            a, b = self._dirty[slot]
            lo, hi = min(a, lo), max(b, hi)
        self._dirty[slot] = (lo, hi)

    def sync(self) -> None:
        """Bring the device block table up to date (changed row segments only)."""
        if self.table_dev is not self.table_cpu:
            for slot, (lo, hi) in self._dirty.items():
                piece = self._staging.take(hi - lo) if self._staging is not None else None
                if piece is None:
                    self.table_dev[slot, lo:hi].copy_(self.table_cpu[slot, lo:hi])
                else:
                    # through pinned memory, in stream order, without waiting: the host's table may
                    # change again (a trim, a freed slot) before the device has taken this piece
                    piece.copy_(self.table_cpu[slot, lo:hi])
                    self.table_dev[slot, lo:hi].copy_(piece, non_blocking=True)
        self._dirty.clear()


class SequenceCache:
    """Slots, page groups and the state area of one model instance."""

    def __init__(self, needs: Dict[int, CacheNeed], states: Dict[object, StateNeed], max_tokens: int,
                 max_seq_len: Optional[int] = None, n_slots: Optional[int] = None,
                 page_tokens: int = PAGE_TOKENS, dtype: Optional[torch.dtype] = torch.float32, device="cpu"):
        if max_tokens <= 0:
            raise CacheError(f"the cache needs room for at least one token, got {max_tokens}")
        self.page_tokens = page_tokens
        self.device = torch.device(device)
        n_pages = -(-max_tokens // page_tokens)
        self.n_pages = n_pages
        if n_slots is None:
            n_slots = n_pages
        self.slots = SlotAllocator(n_slots)
        self.n_slots = n_slots
        if max_seq_len is None:
            max_seq_len = n_pages * page_tokens
        max_pages_per_seq = min(n_pages, -(-max_seq_len // page_tokens))
        self.max_seq_len = max_pages_per_seq * page_tokens
        self.lengths: List[int] = [0] * n_slots
        # group units by equal needs, in order of first appearance
        by_need: Dict[CacheNeed, List[int]] = {}
        for unit, need in needs.items():
            by_need.setdefault(need, []).append(unit)
        self.groups: List[CacheGroup] = [
            CacheGroup(need, units, n_pages, n_slots, max_pages_per_seq, page_tokens, dtype, device)
            for need, units in by_need.items()]
        self.group_of_unit: Dict[int, CacheGroup] = {u: g for g in self.groups for u in g.unit_ids}
        # fixed-size state: one row of bytes per slot, a typed view per owner
        self._state_views: Dict[object, torch.Tensor] = {}
        off = 0
        layout = []
        for key, need in states.items():
            n = 1
            for s in need.shape:
                n *= s
            nbytes = n * torch.empty((), dtype=need.dtype).element_size()
            layout.append((key, need, off, nbytes))
            off += -(-nbytes // 16) * 16
        self.state_bytes_per_slot = off
        self.state_arena = torch.zeros((n_slots, max(off, 16)), dtype=torch.uint8, device=self.device)
        for key, need, o, nbytes in layout:
            self._state_views[key] = self.state_arena[:, o:o + nbytes].view(need.dtype).view((n_slots,) + tuple(need.shape))

    # -- slots -----------------------------------------------------------------------
    def alloc_slot(self) -> int:
        s = self.slots.alloc()
        self.lengths[s] = 0
        if self.state_bytes_per_slot:
            self.state_arena[s].zero_()
        return s

    def free_slot(self, slot: int) -> None:
        self.slots.free(slot)          # raises on a double free before anything is touched
        for g in self.groups:
            g.release(slot)
        self.lengths[slot] = 0

    def length(self, slot: int) -> int:
        self.slots.check_live(slot)
        return self.lengths[slot]

    # -- a step: reserve, then commit --------------------------------------------------
    def reserve(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        """Pages for `new_tokens[i]` more tokens of `slots[i]`, for all or for none."""
        if len(set(slots)) != len(slots):
            raise CacheError("a slot appears twice in one step")
        for s in slots:
            self.slots.check_live(s)
        for g in self.groups:
            need = 0
            for s, n in zip(slots, new_tokens):
                new_len = self.lengths[s] + n
                if new_len > self.max_seq_len:
                    raise CacheError(f"slot {s}: {new_len} tokens exceed the cache's longest sequence {self.max_seq_len}")
                need += g.pages_needed(s, new_len)
            if need > g.pool.free_count:
                raise CacheError(f"out of cache pages: the step needs {need}, {g.pool.free_count} of "
                                 f"{g.pool.n_pages} are free")
        for g in self.groups:
            for s, n in zip(slots, new_tokens):
                g.grow(s, self.lengths[s] + n)
            g.sync()

    def pages_held(self, slots: Sequence[int]) -> List[List[int]]:
        """Per group the number of page entries each of `slots` has now, in their order (what
        `release_reserved` rolls back to).  Slots that are not live count as holding none:
        `reserve` refuses them before it takes anything."""
        n = self.n_slots
        return [[len(g.pages[s]) if isinstance(s, int) and 0 <= s < n else 0 for s in slots] for g in self.groups]

    def release_reserved(self, slots: Sequence[int], held: List[List[int]]) -> None:
        """Undo a `reserve` that no `commit` follows: pages the slots took since `held` was
        read (`pages_held` of the same slots) go back to their pools."""
        for g, before in zip(self.groups, held):
            for s, had in zip(slots, before):
                if not (isinstance(s, int) and 0 <= s < self.n_slots):
                    continue
                extra = g.pages[s][had:]
                if extra:
                    g.pool.free([p for p in extra if p >= 0])
                    g.table_cpu[s, had:len(g.pages[s])] = -1
                    g._mark(s, had, len(g.pages[s]))
                    del g.pages[s][had:]
            g.sync()

    def commit(self, slots: Sequence[int], new_tokens: Sequence[int]) -> None:
        for s, n in zip(slots, new_tokens):
            self.lengths[s] += n
            for g in self.groups:
                g.trim(s, self.lengths[s])

    # -- views for parts ---------------------------------------------------------------
    def unit_storage(self, unit: int) -> torch.Tensor:
        return self.group_of_unit[unit].storage_view(unit)

    def unit_group(self, unit: int) -> CacheGroup:
        return self.group_of_unit[unit]

    def state(self, key) -> Optional[torch.Tensor]:
        return self._state_views.get(key)

    def tokens_held(self) -> int:
        return sum(self.lengths[s] for s in self.slots.live_slots())
