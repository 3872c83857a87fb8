"""The cache manager: pages of keys and values with a block table per request, one pool per
group of layers with the same needs, and slots for per-request state of fixed size.

The bookkeeping itself is native (`csrc/runtime.cpp`); this file groups the layers' needs, names
requests and turns error codes into exceptions.  Addressing and pool discipline follow the
reference's `BlockPool` and `BlockTable` (`inferrs-models/src/kv_cache.rs:80-140`, `:154-222`): a
page holds `page_size` token slots, `slot = table[pos // page_size] * page_size + pos %
page_size`; free pages form a FIFO (taken from the front, given back to the back), so the
physical layout of a replayed trace is deterministic.  Beyond the reference: reservation is
all-or-nothing over all groups, layers with a window give pages back once the window has passed
them, and requests own a slot in the fixed-size state arrays of layers that keep such state.

Nothing here touches a GPU; `storage.py` holds the device arrays.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, Iterator, List, Optional, Sequence, Tuple

from .. import native
from ..parts.base import FixedState, PagedKV

RELEASED = native.RELEASED


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


def _fail() -> None:
    raise CacheError(native.last_error())


class _Handle:
    """Owns one native cache manager."""

    def __init__(self, page_size: int, max_seqs: int, windows: Sequence[int], num_pages: Sequence[int]):
        self.lib = native.runtime()
        self.ptr = self.lib.iar_cache_create(page_size, max_seqs, len(windows), native.ints(list(windows)),
                                             native.ints(list(num_pages)))
        if not self.ptr:
            _fail()

    def __del__(self):
        if getattr(self, "ptr", None):
            self.lib.iar_cache_destroy(self.ptr)
            self.ptr = None


class PagePool:
    """Free list with reference counts over pages 0..num_pages-1: a pool of its own when built
    with a number, or a view of one group's pool of a cache manager."""

    def __init__(self, num_pages: int, _handle: Optional[_Handle] = None, _group: int = 0):
        if _handle is None:
            if num_pages < 0:
                raise CacheError(f"num_pages must be >= 0, got {num_pages}")
            _handle = _Handle(1, 1, [-1], [num_pages])
        self._h, self._g = _handle, _group

    @property
    def num_pages(self) -> int:
        return self._h.lib.iar_cache_num_pages(self._h.ptr, self._g)

    @property
    def num_free(self) -> int:
        return self._h.lib.iar_cache_num_free(self._h.ptr, self._g)

    def allocate(self, n: int) -> Optional[List[int]]:
        """n pages from the front of the free list, or None (and nothing taken)."""
        out = native.ints([0] * max(n, 1))
        got = self._h.lib.iar_cache_pool_allocate(self._h.ptr, self._g, n, out)
        if got == native.NO_PAGES:
            return None
        if got < 0:
            _fail()
        return list(out[:n])

    def free(self, pages: Sequence[int]) -> None:
        if self._h.lib.iar_cache_pool_free(self._h.ptr, self._g, native.ints(list(pages)), len(pages)):
            _fail()


class SlotPool:
    """Ids 0..n-1 for per-request state of fixed size; lowest free id first."""

    def __init__(self, num_slots: int, _handle: Optional[_Handle] = None):
        self._h = _handle or _Handle(1, num_slots, [], [])
        self.num_slots = num_slots

    @property
    def num_free(self) -> int:
        return self._h.lib.iar_cache_free_slots(self._h.ptr)

    def allocate(self) -> Optional[int]:
        s = self._h.lib.iar_cache_slot_allocate(self._h.ptr)
        return None if s < 0 else s

    def free(self, slot: int) -> None:
        if self._h.lib.iar_cache_slot_free(self._h.ptr, slot):
            _fail()


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


class _Tables:
    """The block tables of one request, group -> list of pages (a copy: assign a list to change one)."""

    def __init__(self, manager: "CacheManager", key: int):
        self._m, self._k = manager, key

    def __getitem__(self, group: int) -> List[int]:
        h = self._m._h
        n = h.lib.iar_cache_table_size(h.ptr, self._k, group)
        if n < 0:
            _fail()
        out = native.ints([0] * max(n, 1))
        h.lib.iar_cache_table(h.ptr, self._k, group, out, n)
        return list(out[:n])

    def __setitem__(self, group: int, pages: Sequence[int]) -> None:
        h = self._m._h
        if h.lib.iar_cache_set_table(h.ptr, self._k, group, native.ints(list(pages)), len(pages)):
            _fail()

    def __len__(self) -> int:
        return len(self._m.groups)

    def keys(self):
        return range(len(self._m.groups))

    def values(self) -> List[List[int]]:
        return [self[g] for g in self.keys()]


class SequenceCache:
    """What the manager holds for one live request."""

    def __init__(self, manager: "CacheManager", seq_id: Hashable, key: int):
        self._m, self.seq_id, self._k = manager, seq_id, key

    def _get(self, fn) -> int:
        v = fn(self._m._h.ptr, self._k)
        if v < 0:
            _fail()
        return v

    @property
    def length(self) -> int:
        """Tokens whose keys are cached."""
        return self._get(self._m._h.lib.iar_cache_length)

    @property
    def reserved(self) -> int:
        """Tokens reserved beyond `length`."""
        return self._get(self._m._h.lib.iar_cache_reserved)

    @property
    def state_slot(self) -> int:
        return self._get(self._m._h.lib.iar_cache_state_slot)

    @property
    def tables(self) -> _Tables:
        return _Tables(self._m, self._k)


class _Sequences:
    """The live requests by name."""

    def __init__(self, manager: "CacheManager"):
        self._m = manager

    def __contains__(self, seq_id: Hashable) -> bool:
        k = self._m.names.find(seq_id)
        return k is not None and bool(self._m._h.lib.iar_cache_has_sequence(self._m._h.ptr, k))

    def __getitem__(self, seq_id: Hashable) -> SequenceCache:
        if seq_id not in self:
            raise KeyError(seq_id)
        return SequenceCache(self._m, seq_id, self._m.names.find(seq_id))

    def get(self, seq_id: Hashable, default=None):
        return self[seq_id] if seq_id in self else default

    def __len__(self) -> int:
        return self._m._h.lib.iar_cache_num_sequences(self._m._h.ptr)

    def __iter__(self) -> Iterator[Hashable]:
        return iter([n for n in self._m.names.names() if n in self])

    def keys(self):
        return list(self)

    def values(self) -> List[SequenceCache]:
        return [self[n] for n in self]


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
        windows = [-1 if need.window is None else need.window for need, _ in grouped]
        self._h = _Handle(page_size, max_seqs, windows, list(num_pages))
        self.names = native.KeyTable()
        self.groups: List[GroupInfo] = [GroupInfo(i, need, layers, PagePool(0, self._h, i))
                                        for i, (need, layers) in enumerate(grouped)]
        self.layer_group: Dict[int, int] = {l: g.index for g in self.groups for l in g.layers}
        self.slots = SlotPool(max_seqs, self._h)
        self.sequences = _Sequences(self)

    @property
    def handle(self):
        """The native object, for the step builder and the scheduler."""
        return self._h.ptr

    def _key(self, seq_id: Hashable) -> int:
        k = self.names.find(seq_id)
        if k is None or not self._h.lib.iar_cache_has_sequence(self._h.ptr, k):
            raise CacheError(f"request {seq_id!r} is not live")
        return k

    # ---- requests ---------------------------------------------------------------------------
    def add_sequence(self, seq_id: Hashable) -> SequenceCache:
        if seq_id in self.sequences:
            raise CacheError(f"request {seq_id!r} is already live")
        k = self.names.key(seq_id)
        if self._h.lib.iar_cache_add_sequence(self._h.ptr, k) < 0:
            self.names.drop(seq_id)
            _fail()
        return SequenceCache(self, seq_id, k)

    def free_sequence(self, seq_id: Hashable) -> None:
        k = self._key(seq_id)
        if self._h.lib.iar_cache_free_sequence(self._h.ptr, k):
            _fail()
        self.names.drop(seq_id)

    def length(self, seq_id: Hashable) -> int:
        return self._h.lib.iar_cache_length(self._h.ptr, self._key(seq_id))

    # ---- pages ------------------------------------------------------------------------------
    def can_reserve(self, asks: Sequence[Tuple[Hashable, int]]) -> bool:
        ks = [self._key(s) for s, _ in asks]
        return bool(self._h.lib.iar_cache_can_reserve(self._h.ptr, len(ks), native.keys(ks),
                                                      native.ints([n for _, n in asks])))

    def reserve(self, seq_id: Hashable, n_new: int) -> bool:
        """Pages for the next `n_new` tokens in every group, or nothing at all."""
        code = self._h.lib.iar_cache_reserve(self._h.ptr, self._key(seq_id), n_new)
        if code == native.NO_PAGES:
            return False
        if code:
            _fail()
        return True

    def commit(self, seq_id: Hashable, n_new: int) -> None:
        """`n_new` reserved tokens are now cached; pages that every window has passed go back."""
        if self._h.lib.iar_cache_commit(self._h.ptr, self._key(seq_id), n_new):
            raise CacheError(f"request {seq_id!r}: {native.last_error()}")

    # ---- whole batches ----------------------------------------------------------------------
    def _keys_of(self, seq_ids: Sequence[Hashable]):
        find = self.names.find
        ks = [find(s) for s in seq_ids]
        if None in ks:
            raise CacheError(f"request {seq_ids[ks.index(None)]!r} is not live")
        return native.keys(ks)

    def all_live(self, seq_ids: Sequence[Hashable]) -> bool:
        find = self.names.find
        ks = [find(s) for s in seq_ids]
        return None not in ks and self._h.lib.iar_cache_count_live(self._h.ptr, len(ks), native.keys(ks)) == len(ks)

    def max_length(self, seq_ids: Sequence[Hashable]) -> int:
        """The greatest cached length among live requests."""
        n = self._h.lib.iar_cache_max_length(self._h.ptr, len(seq_ids), self._keys_of(seq_ids))
        if n < 0:
            _fail()
        return n

    def ensure_reserved(self, asks: Sequence[Tuple[Hashable, int]]) -> bool:
        """Every request holds reservations for at least that many tokens afterwards, or nothing
        was taken for any of them."""
        code = self._h.lib.iar_cache_ensure_reserved(self._h.ptr, len(asks), self._keys_of([s for s, _ in asks]),
                                                     native.ints([n for _, n in asks]))
        if code == native.NO_PAGES:
            return False
        if code:
            _fail()
        return True

    def commit_many(self, commits: Sequence[Tuple[Hashable, int]]) -> None:
        if self._h.lib.iar_cache_commit_many(self._h.ptr, len(commits), self._keys_of([s for s, _ in commits]),
                                             native.ints([n for _, n in commits])):
            _fail()

    def slot_ids(self, seq_id: Hashable, group: int, start: int, n: int) -> List[int]:
        """Physical slots of positions start..start+n (`kv_cache.rs:183-192`)."""
        out = native.ints([0] * max(n, 1))
        if self._h.lib.iar_cache_slot_ids(self._h.ptr, self._key(seq_id), group, start, n, out):
            raise CacheError(f"request {seq_id!r}: {native.last_error()}")
        return list(out[:n])

    def check_invariants(self) -> None:
        """No page lost, held twice or free while held.  For tests."""
        if self._h.lib.iar_cache_check_invariants(self._h.ptr):
            _fail()
