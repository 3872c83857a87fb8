"""The cache manager: pages of keys and values with a block table per request, one pool per
group of layers with the same needs, and slots for per-request state of fixed size.

Addressing and pool discipline follow the reference's `BlockPool` and `BlockTable`
(`inferrs-models/src/kv_cache.rs:80-140`, `:154-222`): a page holds `page_size` token
slots, `slot = table[pos // page_size] * page_size + pos % page_size`; free pages form a
FIFO (taken from the front, given back to the back), so the physical layout of a replayed
trace is deterministic.  Beyond the reference: reservation is all-or-nothing over all
groups, layers with a window give pages back once the window has passed them, and
requests own a slot in the fixed-size state arrays of layers that keep such state.

The bookkeeping in this file is host-only and runs without a GPU; `storage.py` holds the
device arrays.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..parts.base import FixedState, PagedKV

RELEASED = -1


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


class PagePool:
    """Free list with reference counts over pages 0..num_pages-1."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise CacheError(f"num_pages must be >= 0, got {num_pages}")
        self.num_pages = num_pages
        self._free: Deque[int] = deque(range(num_pages))
        self._refs: List[int] = [0] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, n: int) -> Optional[List[int]]:
        """n pages from the front of the free list, or None (and nothing taken)."""
        if n < 0:
            raise CacheError(f"cannot allocate {n} pages")
        if len(self._free) < n:
            return None
        out = [self._free.popleft() for _ in range(n)]
        for p in out:
            if self._refs[p] != 0:
                raise CacheError(f"page {p} was on the free list while still held")
            self._refs[p] = 1
        return out

    def free(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not (0 <= p < self.num_pages):
                raise CacheError(f"page {p} does not belong to this pool of {self.num_pages}")
            if self._refs[p] <= 0:
                raise CacheError(f"page {p} freed twice")
            self._refs[p] -= 1
            if self._refs[p] == 0:
                self._free.append(p)

    def held(self) -> List[int]:
        return [p for p, r in enumerate(self._refs) if r > 0]


class SlotPool:
    """Ids 0..n-1 for per-request state of fixed size; lowest free id first."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free: List[int] = list(range(num_slots - 1, -1, -1))
        self._held = [False] * num_slots

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> Optional[int]:
        if not self._free:
            return None
        s = self._free.pop()
        self._held[s] = True
        return s

    def free(self, slot: int) -> None:
        if not (0 <= slot < self.num_slots) or not self._held[slot]:
            raise CacheError(f"state slot {slot} freed twice or never held")
        self._held[slot] = False
        self._free.append(slot)
        self._free.sort(reverse=True)


@dataclass
class GroupInfo:
    """Layers whose caches have the same geometry share pages of one pool."""
    index: int
    need: PagedKV
    layers: List[int]
    pool: PagePool


@dataclass
class StateInfo:
    layer: int
    need: FixedState


@dataclass
class SequenceCache:
    seq_id: Hashable
    length: int = 0                                   # tokens whose keys are cached
    tables: Dict[int, List[int]] = field(default_factory=dict)   # group -> logical page -> physical
    state_slot: int = -1
    reserved: int = 0                                 # tokens reserved beyond `length`


def group_layers(needs: Dict[int, object]) -> Tuple[List[Tuple[PagedKV, List[int]]], List[StateInfo]]:
    """Cache-owning layers -> (paged groups in order of first layer, state layers)."""
    groups: Dict[PagedKV, List[int]] = {}
    states: List[StateInfo] = []
    for layer in sorted(needs):
        need = needs[layer]
        if need is None:
            continue
        if isinstance(need, PagedKV):
            groups.setdefault(need, []).append(layer)
        elif isinstance(need, FixedState):
            states.append(StateInfo(layer, need))
        else:
            raise CacheError(f"layer {layer}: unknown cache need {need!r}")
    return list(groups.items()), states


class CacheManager:
    def __init__(self, needs: Dict[int, object], page_size: int, num_pages, max_seqs: int):
        """`needs`: cache-owning layer -> PagedKV | FixedState | None.
        `num_pages`: an int for every group, or a list with one entry per group."""
        if page_size < 1:
            raise CacheError(f"page_size must be >= 1, got {page_size}")
        if max_seqs < 1:
            raise CacheError(f"max_seqs must be >= 1, got {max_seqs}")
        self.page_size = page_size
        self.max_seqs = max_seqs
        grouped, self.states = group_layers(needs)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(grouped)
        if len(num_pages) != len(grouped):
            raise CacheError(f"{len(grouped)} cache groups but {len(num_pages)} page counts")
        self.groups: List[GroupInfo] = [
            GroupInfo(i, need, layers, PagePool(n)) for i, ((need, layers), n) in enumerate(zip(grouped, num_pages))]
        self.layer_group: Dict[int, int] = {l: g.index for g in self.groups for l in g.layers}
        self.slots = SlotPool(max_seqs)
        self.sequences: Dict[Hashable, SequenceCache] = {}

    # ---- requests ---------------------------------------------------------------------------
    def add_sequence(self, seq_id: Hashable) -> SequenceCache:
        if seq_id in self.sequences:
            raise CacheError(f"request {seq_id!r} is already live")
        slot = self.slots.allocate()
        if slot is None:
            raise CacheError(f"all {self.max_seqs} request slots are in use")
        seq = SequenceCache(seq_id, 0, {g.index: [] for g in self.groups}, slot)
        self.sequences[seq_id] = seq
        return seq

    def free_sequence(self, seq_id: Hashable) -> None:
        seq = self.sequences.pop(seq_id, None)
        if seq is None:
            raise CacheError(f"request {seq_id!r} is not live")
        for g in self.groups:
            g.pool.free([p for p in seq.tables[g.index] if p != RELEASED])
        self.slots.free(seq.state_slot)

    # ---- pages ------------------------------------------------------------------------------
    def _pages_for(self, length: int) -> int:
        return -(-length // self.page_size)

    def pages_needed(self, seq_id: Hashable, n_new: int) -> List[int]:
        """New pages per group to hold `n_new` more tokens than are cached or reserved."""
        seq = self.sequences[seq_id]
        total = self._pages_for(seq.length + seq.reserved + n_new)
        return [max(0, total - len(seq.tables[g.index])) for g in self.groups]

    def can_reserve(self, asks: Sequence[Tuple[Hashable, int]]) -> bool:
        want = [0] * len(self.groups)
        for seq_id, n_new in asks:
            for i, n in enumerate(self.pages_needed(seq_id, n_new)):
                want[i] += n
        return all(want[i] <= g.pool.num_free for i, g in enumerate(self.groups))

    def reserve(self, seq_id: Hashable, n_new: int) -> bool:
        """Pages for the next `n_new` tokens in every group, or nothing at all."""
        if n_new < 0:
            raise CacheError(f"cannot reserve {n_new} tokens")
        seq = self.sequences[seq_id]
        need = self.pages_needed(seq_id, n_new)
        if any(n > g.pool.num_free for n, g in zip(need, self.groups)):
            return False
        for n, g in zip(need, self.groups):
            got = g.pool.allocate(n)
            assert got is not None
            seq.tables[g.index].extend(got)
        seq.reserved += n_new
        return True

    def commit(self, seq_id: Hashable, n_new: int) -> None:
        """`n_new` reserved tokens are now cached; pages that every window has passed go back."""
        seq = self.sequences[seq_id]
        if n_new > seq.reserved:
            raise CacheError(f"request {seq_id!r}: commit of {n_new} tokens but {seq.reserved} reserved")
        seq.length += n_new
        seq.reserved -= n_new
        for g in self.groups:
            w = g.need.window
            if w is None:
                continue
            # The next query sits at position `length` and reads keys > length - w.
            first_needed = max(0, seq.length - w + 1)
            table = seq.tables[g.index]
            passed = [i for i in range(min(first_needed // self.page_size, len(table))) if table[i] != RELEASED]
            g.pool.free([table[i] for i in passed])
            for i in passed:
                table[i] = RELEASED

    def slot_ids(self, seq_id: Hashable, group: int, start: int, n: int) -> List[int]:
        """Physical slots of positions start..start+n (`kv_cache.rs:183-192`)."""
        table = self.sequences[seq_id].tables[group]
        ps = self.page_size
        out = []
        for pos in range(start, start + n):
            page = table[pos // ps]
            if page == RELEASED:
                raise CacheError(f"request {seq_id!r}: position {pos} lies in a released page")
            out.append(page * ps + pos % ps)
        return out

    def check_invariants(self) -> None:
        """No page lost, held twice or free while held.  For tests."""
        for g in self.groups:
            held = sorted(p for s in self.sequences.values() for p in s.tables[g.index] if p != RELEASED)
            if len(held) != len(set(held)):
                raise CacheError(f"group {g.index}: a page is held twice: {held}")
            if held != g.pool.held():
                raise CacheError(f"group {g.index}: tables hold {held}, pool says {g.pool.held()}")
            free = sorted(g.pool._free)
            if len(free) != len(set(free)) or set(free) & set(held):
                raise CacheError(f"group {g.index}: free list {free} overlaps held pages or repeats")
            if len(free) + len(held) != g.pool.num_pages:
                raise CacheError(f"group {g.index}: {len(free)} free + {len(held)} held != {g.pool.num_pages}")
        slots = [s.state_slot for s in self.sequences.values()]
        if len(slots) != len(set(slots)):
            raise CacheError(f"a state slot is held twice: {slots}")
