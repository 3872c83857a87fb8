"""What one step hands to the model: the flattened tokens of all requests in the batch and,
per cache group, where their keys go and where earlier keys lie.

The reference builds the equivalent once per pass for ONE sequence (`PagedPassCache::build`,
`inferrs-models/src/models/attention_utils.rs:252-283`: slot ids for the new tokens, a causal
mask).  Here a step holds any mix of requests, each with a span of new tokens starting at
its cached length, and no mask is built: kernels derive causality from `positions`.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Any, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import native
from ..cache.manager import CacheManager


@dataclass
class GroupStep:
    """Per cache group: `slots[i]` = page * page_size + offset for token i's key and value;
    `block_table[s]` = the pages of request s in logical order."""
    page_size: int
    slots: torch.Tensor          # int32 [n_tokens]
    block_table: torch.Tensor    # int32 [n_seqs, max_pages]


@dataclass
class StepContext:
    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor      # int32 [n_tokens]
    positions: torch.Tensor      # int32 [n_tokens]   absolute position of each token
    token_seq: torch.Tensor      # int32 [n_tokens]   row of the batch each token belongs to
    cu_tokens: torch.Tensor      # int32 [n_seqs + 1] token spans: request s owns cu[s]..cu[s+1]
    state_slots: torch.Tensor    # int32 [n_seqs]     row of the fixed-size state arrays
    want_rows: torch.Tensor      # int32 [n_want]     tokens whose logits are returned
    groups: List[GroupStep]
    # host copies, for launch decisions and for parts that loop on the host
    q_lens: List[int] = field(default_factory=list)
    kv_starts: List[int] = field(default_factory=list)
    state_slots_host: List[int] = field(default_factory=list)
    max_q_len: int = 0
    max_kv_len: int = 0
    n_single: int = 0            # the first n_single requests bring one token each (they come first)
    max_kv_single: int = 0       # the greatest length among those, after the step
    max_kv_multi: int = 0        # and among the others
    stream: Optional[torch.Tensor] = None   # set by a block around a part that may add its output to it itself
    stream_norm: Any = None                 # and the norm part that will read the stream next
    partial_sums: bool = False              # set by a block whose norms take a part's last product split along k
    _tables: Dict[Any, Any] = field(default_factory=dict)

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1

    def position_table(self, position_part) -> Optional[Any]:
        """The position part's table for this step's tokens, built once per distinct spec."""
        key = position_part.spec
        if key not in self._tables:
            self._tables[key] = position_part.table(self.positions)
        return self._tables[key]


class StepError(ValueError):
    pass


class StepBuilder:
    """Turns (request, its next tokens, wanted places) into a `StepContext`.  The native runtime
    writes every array of the step into a pinned staging buffer (`iar_build_step` in
    `csrc/runtime.cpp`), and one copy takes it to the device."""

    RING = 16

    def __init__(self, cache: CacheManager, device):
        self.cache = cache
        self.device = torch.device(device)
        self._lib = native.runtime()
        # One device buffer (its address is what captured graphs hold) and a ring of pinned host
        # buffers, so that the copies of several steps can be under way at once.
        self._ring: List[torch.Tensor] = []
        self._flat: List[np.ndarray] = []
        self._events: List[Optional[torch.cuda.Event]] = []
        self._next = 0
        self._dev: Optional[torch.Tensor] = None
        self._meta = (ctypes.c_int * 16)()
        self.generation = 0                # grows when the device staging buffer moves

    def _staging(self, n: int) -> Tuple[torch.Tensor, torch.Tensor, int]:
        if self._dev is None or self._dev.numel() < n:
            size = 1 << max(12, (n - 1).bit_length())
            torch.cuda.synchronize(self.device)
            self._ring = [torch.empty(size, dtype=torch.int32, pin_memory=True) for _ in range(self.RING)]
            self._flat = [t.numpy() for t in self._ring]
            self._events = [None] * self.RING
            self._dev = torch.empty(size, dtype=torch.int32, device=self.device)
            self.generation += 1
        slot = self._next
        self._next = (slot + 1) % self.RING
        if self._events[slot] is not None:
            self._events[slot].synchronize()      # that copy has left the host buffer
        return self._ring[slot], self._dev, slot

    def build(self, entries: Sequence[Tuple[Hashable, Sequence[int], Sequence[int]]],
              pad_pages: Optional[int] = None, advance: int = 0, skip_tokens: bool = False) -> StepContext:
        """`entries`: (request, tokens, want).  The requests are live and hold pages for the
        positions `length .. length + len(tokens)`.  Requests with a single token are put first (in
        their order), the others after them: mixers can then treat the two runs apart; wanted rows
        keep the callers' order.  `pad_pages`: width of the block tables (at least what the longest
        request needs); with it the place of every array in the staging buffer depends on the
        counts of tokens, requests and wanted rows only.  `advance`: the requests are taken to be
        that many tokens longer than the cache manager says (steps that are queued before the
        steps ahead of them are committed).  `skip_tokens`: the token ids are not copied to the
        device (they are written there by the step before)."""
        s_count = len(entries)
        names = self.cache.names
        key_list = []
        for e in entries:
            k = names.find(e[0])
            if k is None:
                raise StepError(f"request {e[0]!r} is not live")
            key_list.append(k)
        q_given = [len(e[1]) for e in entries]
        n = sum(q_given)
        want_counts = [len(e[2]) for e in entries]
        n_want = sum(want_counts)
        if n == s_count:
            tokens = native.ints([e[1][0] for e in entries])
        elif n <= 256:
            tokens = native.ints([t for e in entries for t in e[1]])
        else:
            tokens = np.concatenate([np.asarray(e[1], dtype=np.int32) for e in entries])
        want = native.ints([w for e in entries for w in e[2]])
        c_keys, c_q, c_wc = native.keys(key_list), native.ints(q_given), native.ints(want_counts)
        pad = pad_pages if pad_pages is not None else 0
        lib, handle = self._lib, self.cache.handle
        total = lib.iar_step_words(handle, s_count, c_keys, c_q, n_want, pad, advance)
        if total < 0:
            raise StepError(native.last_error())
        host, dev, slot = self._staging(max(int(total), 1))
        flat = self._flat[slot]
        order = (ctypes.c_int * max(s_count, 1))()
        meta = self._meta
        token_ptr = tokens.ctypes.data if isinstance(tokens, np.ndarray) else ctypes.addressof(tokens)
        if lib.iar_build_step(handle, s_count, c_keys, c_q, token_ptr, c_wc, want, pad, advance,
                              host.data_ptr(), host.numel(), meta, order):
            raise StepError(native.last_error())
        total, max_pages, n_groups = meta[0], meta[4], meta[10]
        first = n if skip_tokens else 0                 # the token ids come first
        dev[first:total].copy_(host[first:total], non_blocking=True)
        self._events[slot] = torch.cuda.Event()
        self._events[slot].record()
        off = 0
        views = []
        for sz in (n, n, n, s_count + 1, s_count, n_want):
            views.append(dev[off:off + sz])
            off += sz
        cu_off, slot_off = 3 * n, 3 * n + s_count + 1
        groups = []
        for _ in range(n_groups):
            slots = dev[off:off + n]
            off += n
            groups.append(GroupStep(self.cache.page_size, slots, dev[off:off + s_count * max_pages].view(s_count, max_pages)))
            off += s_count * max_pages
        cu = flat[cu_off:cu_off + s_count]
        return StepContext(
            n_tokens=n, n_seqs=s_count, token_ids=views[0], positions=views[1], token_seq=views[2],
            cu_tokens=views[3], state_slots=views[4], want_rows=views[5], groups=groups,
            q_lens=[q_given[order[j]] for j in range(s_count)], kv_starts=flat[n + cu].tolist(),
            state_slots_host=flat[slot_off:slot_off + s_count].tolist(),
            max_q_len=meta[5], max_kv_len=meta[6], n_single=meta[7], max_kv_single=meta[8], max_kv_multi=meta[9])
