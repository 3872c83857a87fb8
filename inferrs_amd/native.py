"""The door to the host runtime library (cache manager, step assembly, scheduler: plain C++ under
`csrc/runtime.cpp`).  It is compiled on first use when no built library is found; it needs no
GPU.  Requests are named by 64-bit keys on the C side; `KeyTable` maps the caller's hashable
names to keys."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_longlong, c_void_p
from typing import Dict, Hashable, Optional

ERROR, NO_PAGES, RELEASED = -1, -2, -1
_LIB: Optional[ctypes.CDLL] = None
_PATH: Optional[str] = None

_PI, _PK = POINTER(c_int), POINTER(c_int64)
_SIGNATURES = {
    "iar_last_error": (c_char_p, []),
    "iar_abi_version": (c_int, []),
    "iar_cache_create": (c_void_p, [c_int, c_int, c_int, _PI, _PI]),
    "iar_cache_destroy": (None, [c_void_p]),
    "iar_cache_add_sequence": (c_int, [c_void_p, c_int64]),
    "iar_cache_free_sequence": (c_int, [c_void_p, c_int64]),
    "iar_cache_has_sequence": (c_int, [c_void_p, c_int64]),
    "iar_cache_num_sequences": (c_int, [c_void_p]),
    "iar_cache_length": (c_int, [c_void_p, c_int64]),
    "iar_cache_reserved": (c_int, [c_void_p, c_int64]),
    "iar_cache_state_slot": (c_int, [c_void_p, c_int64]),
    "iar_cache_reserve": (c_int, [c_void_p, c_int64, c_int]),
    "iar_cache_can_reserve": (c_int, [c_void_p, c_int, _PK, _PI]),
    "iar_cache_commit": (c_int, [c_void_p, c_int64, c_int]),
    "iar_cache_count_live": (c_int, [c_void_p, c_int, _PK]),
    "iar_cache_max_length": (c_int, [c_void_p, c_int, _PK]),
    "iar_cache_ensure_reserved": (c_int, [c_void_p, c_int, _PK, _PI]),
    "iar_cache_commit_many": (c_int, [c_void_p, c_int, _PK, _PI]),
    "iar_cache_table_size": (c_int, [c_void_p, c_int64, c_int]),
    "iar_cache_table": (c_int, [c_void_p, c_int64, c_int, _PI, c_int]),
    "iar_cache_set_table": (c_int, [c_void_p, c_int64, c_int, _PI, c_int]),
    "iar_cache_slot_ids": (c_int, [c_void_p, c_int64, c_int, c_int, c_int, _PI]),
    "iar_cache_num_free": (c_int, [c_void_p, c_int]),
    "iar_cache_num_pages": (c_int, [c_void_p, c_int]),
    "iar_cache_free_slots": (c_int, [c_void_p]),
    "iar_cache_pool_allocate": (c_int, [c_void_p, c_int, c_int, _PI]),
    "iar_cache_pool_free": (c_int, [c_void_p, c_int, _PI, c_int]),
    "iar_cache_slot_allocate": (c_int, [c_void_p]),
    "iar_cache_slot_free": (c_int, [c_void_p, c_int]),
    "iar_cache_check_invariants": (c_int, [c_void_p]),
    "iar_build_step": (c_int, [c_void_p, c_int, _PK, _PI, c_void_p, _PI, _PI, c_int, c_int, c_void_p,
                               c_longlong, _PI, _PI]),
    "iar_step_words": (c_longlong, [c_void_p, c_int, _PK, _PI, c_int, c_int, c_int]),
    "iar_sched_create": (c_void_p, [c_void_p, c_int, c_int, c_int, c_int, _PI, c_int]),
    "iar_sched_set_row_multiple": (c_int, [c_void_p, c_int]),
    "iar_sched_destroy": (None, [c_void_p]),
    "iar_sched_add": (c_int, [c_void_p, c_int64, _PI, c_int, c_int, c_int, _PI, c_int]),
    "iar_sched_adopt": (c_int, [c_void_p, c_int64, _PI, c_int, c_int, c_int, c_int, _PI, c_int]),
    "iar_sched_num_waiting": (c_int, [c_void_p]),
    "iar_sched_num_running": (c_int, [c_void_p]),
    "iar_sched_waiting": (c_int, [c_void_p, _PK, c_int]),
    "iar_sched_running": (c_int, [c_void_p, _PK, c_int]),
    "iar_sched_plan": (c_int, [c_void_p]),
    "iar_sched_plan_entries": (c_int, [c_void_p, _PK, _PI, _PI, _PI]),
    "iar_sched_plan_tokens": (c_int, [c_void_p, c_int, _PI, c_int]),
    "iar_sched_plan_preempted": (c_int, [c_void_p, _PK, c_int]),
    "iar_sched_plan_failed": (c_int, [c_void_p, _PK, c_int]),
    "iar_sched_failure": (c_char_p, [c_void_p, c_int64]),
    "iar_sched_commit": (c_int, [c_void_p, _PI, c_int, _PK, _PI, c_int]),
    "iar_sched_commit_decode": (c_int, [c_void_p, c_int, _PK, _PI, _PK, _PI, c_int]),
    "iar_sched_request_state": (c_int, [c_void_p, c_int64, _PI]),
    "iar_sched_request_output": (c_int, [c_void_p, c_int64, _PI, c_int]),
    "iar_sched_finish": (c_int, [c_void_p, c_int64]),
    "iar_sched_forget": (c_int, [c_void_p, c_int64]),
}


def runtime() -> ctypes.CDLL:
    global _LIB, _PATH
    if _LIB is not None:
        return _LIB
    from .ops import build
    path = build.library_path("runtime") or build.build("runtime", verbose=True)
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    if lib.iar_abi_version() != 1:
        raise RuntimeError(f"{path}: unexpected ABI version {lib.iar_abi_version()}")
    _LIB, _PATH = lib, path
    return lib


def runtime_file() -> Optional[str]:
    return _PATH


def last_error() -> str:
    return runtime().iar_last_error().decode("utf-8", "replace")


def ints(values) -> ctypes.Array:
    return (c_int * len(values))(*values)


def keys(values) -> ctypes.Array:
    return (c_int64 * len(values))(*values)


class KeyTable:
    """Hashable request names <-> the 64-bit keys of the C side.  A name keeps its key until it
    is dropped; `pin` keeps it over a time in which the request holds no cache entry (it waits
    in a scheduler's line)."""

    def __init__(self):
        self._key: Dict[Hashable, int] = {}
        self._name: Dict[int, Hashable] = {}
        self._pins: Dict[Hashable, int] = {}
        self._next = 1

    def key(self, name: Hashable) -> int:
        k = self._key.get(name)
        if k is None:
            k = self._next
            self._next += 1
            self._key[name] = k
            self._name[k] = name
        return k

    def find(self, name: Hashable) -> Optional[int]:
        return self._key.get(name)

    def name(self, key: int) -> Hashable:
        return self._name[key]

    def names(self):
        return list(self._key)

    def pin(self, name: Hashable) -> int:
        self._pins[name] = self._pins.get(name, 0) + 1
        return self.key(name)

    def unpin(self, name: Hashable, live: bool) -> None:
        n = self._pins.get(name, 0) - 1
        if n > 0:
            self._pins[name] = n
        else:
            self._pins.pop(name, None)
            if not live:
                self.drop(name)

    def drop(self, name: Hashable) -> None:
        """Forget the name unless somebody pinned it."""
        if name in self._pins:
            return
        k = self._key.pop(name, None)
        if k is not None:
            del self._name[k]
