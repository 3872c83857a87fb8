"""What one step hands to the model: the flattened tokens of all requests in the batch and,
per cache group, where their keys go and where earlier keys lie.

The reference builds the equivalent once per pass for ONE sequence (`PagedPassCache::build`,
`inferrs-models/src/models/attention_utils.rs:252-283`: slot ids for the new tokens, a causal
mask).  Here a step holds any mix of requests, each with a span of new tokens starting at
its cached length, and no mask is built: kernels derive causality from `positions`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import RELEASED, CacheManager


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
    """Turns (request, its next tokens, wanted places) into a `StepContext`: everything the
    kernels need goes to the device in one copy from a pinned staging buffer."""

    def __init__(self, cache: CacheManager, device):
        self.cache = cache
        self.device = torch.device(device)
        # One device buffer (its address is what captured graphs hold) and a ring of pinned host
        # buffers, so that the copies of several steps can be under way at once.
        self._ring: List[torch.Tensor] = []
        self._events: List[Optional[torch.cuda.Event]] = []
        self._next = 0
        self._dev: Optional[torch.Tensor] = None
        self._rows: Dict[Any, list] = {}
        self.generation = 0                # grows when the device staging buffer moves

    RING = 16

    def _staging(self, n: int) -> Tuple[torch.Tensor, torch.Tensor, int]:
        if self._dev is None or self._dev.numel() < n:
            size = 1 << max(12, (n - 1).bit_length())
            torch.cuda.synchronize(self.device)
            self._ring = [torch.empty(size, dtype=torch.int32, pin_memory=True) for _ in range(self.RING)]
            self._events = [None] * self.RING
            self._dev = torch.empty(size, dtype=torch.int32, device=self.device)
            self.generation += 1
        slot = self._next
        self._next = (slot + 1) % self.RING
        if self._events[slot] is not None:
            self._events[slot].synchronize()      # that copy has left the host buffer
        return self._ring[slot], self._dev, slot

    def _table_row(self, group: int, seq, need: int) -> np.ndarray:
        """The request's pages of one group as an int32 array, kept between steps and extended
        by the pages that were added since (tables only grow, except where a window releases)."""
        table = seq.tables[group]
        if self.cache.groups[group].need.window is not None:
            return np.asarray(table, dtype=np.int32)
        key = (group, seq.seq_id)
        hit = self._rows.get(key)
        if hit is None or hit[0] is not seq or hit[1].size < len(table):
            arr = np.zeros(max(64, 2 * len(table), need), dtype=np.int32)
            arr[:len(table)] = table
            if len(self._rows) > 4 * max(len(self.cache.sequences), 16):
                live = self.cache.sequences
                self._rows = {k: v for k, v in self._rows.items() if live.get(k[1]) is v[0]}
            self._rows[key] = [seq, arr, len(table)]
            return arr[:len(table)]
        _, arr, filled = hit
        if len(table) > filled:
            arr[filled:len(table)] = table[filled:]
            hit[2] = len(table)
        return arr[:len(table)]

    def build(self, entries: Sequence[Tuple[Hashable, Sequence[int], Sequence[int]]],
              pad_pages: Optional[int] = None, advance: int = 0, skip_tokens: bool = False) -> StepContext:
        """`entries`: (request, tokens, want).  The requests are live and hold pages for the
        positions `length .. length + len(tokens)`.  `pad_pages`: width of the block tables (at
        least what the longest request needs); with it the place of every array in the staging
        buffer depends on the counts of tokens, requests and wanted rows only.  `advance`: the
        requests are taken to be that many tokens longer than the cache manager says (steps that
        are queued before the steps ahead of them are committed).  `skip_tokens`: the token ids
        are not copied to the device (they are written there by the step before)."""
        ps = self.cache.page_size
        # Requests with a single token go first (in their order), the others after them: mixers
        # can then treat the two runs apart.  Wanted rows keep the callers' order.
        order = sorted(range(len(entries)), key=lambda i: len(entries[i][1]) != 1)
        rank = {orig: new for new, orig in enumerate(order)}
        given = entries
        entries = [given[i] for i in order]
        seqs = [self.cache.sequences[e[0]] for e in entries]
        q_lens = [len(e[1]) for e in entries]
        starts = [s.length + advance for s in seqs]
        n, s_count = sum(q_lens), len(entries)
        n_groups = len(self.cache.groups)
        max_pages = max(1, max(-(-(st + q) // ps) for st, q in zip(starts, q_lens)))
        if pad_pages is not None:
            if pad_pages < max_pages:
                raise StepError(f"block tables of {pad_pages} pages are too narrow for {max_pages}")
            max_pages = pad_pages
        cu = np.zeros(s_count + 1, dtype=np.int64)
        np.cumsum(q_lens, out=cu[1:])
        if n == s_count:                                   # one token a request
            token_ids = np.fromiter((e[1][0] for e in entries), dtype=np.int32, count=n)
            positions = np.asarray(starts, dtype=np.int32)
            token_seq = np.arange(s_count, dtype=np.int32)
        else:
            token_ids = np.concatenate([np.asarray(e[1], dtype=np.int32) for e in entries])
            positions = np.concatenate([np.arange(st, st + q, dtype=np.int32) for st, q in zip(starts, q_lens)])
            token_seq = np.repeat(np.arange(s_count, dtype=np.int32), q_lens)
        want = np.asarray([cu[rank[i]] + w for i, e in enumerate(given) for w in e[2]], dtype=np.int32)
        state_slots = np.asarray([s.state_slot for s in seqs], dtype=np.int32)
        tables, slots = [], []
        for g in range(n_groups):
            bt = np.zeros((s_count, max_pages), dtype=np.int32)
            for i, s in enumerate(seqs):
                need = -(-(starts[i] + q_lens[i]) // ps)
                row = self._table_row(g, s, need)
                if row.size < need:
                    raise StepError(f"request {s.seq_id!r} holds {row.size} pages, too few for "
                                    f"{starts[i] + q_lens[i]} tokens")
                bt[i, :min(row.size, max_pages)] = row[:max_pages]
            pages_of_token = bt[token_seq, positions // ps]
            if n and (pages_of_token == RELEASED).any():
                raise StepError("a new token falls into a page that was already released")
            slots.append((pages_of_token * ps + positions % ps).astype(np.int32))
            np.maximum(bt, 0, out=bt)                 # released pages are never read
            tables.append(bt)

        parts = [token_ids, positions, token_seq, cu.astype(np.int32), state_slots, want]
        for g in range(n_groups):
            parts += [slots[g], tables[g].reshape(-1)]
        sizes = [p.size for p in parts]
        total = sum(sizes)
        host, dev, slot = self._staging(max(total, 1))
        flat = host.numpy()
        off, views = 0, []
        for p, sz in zip(parts, sizes):
            flat[off:off + sz] = p
            views.append(dev[off:off + sz])
            off += sz
        first = n if skip_tokens else 0                 # the token ids come first
        dev[first:total].copy_(host[first:total], non_blocking=True)
        self._events[slot] = torch.cuda.Event()
        self._events[slot].record()
        groups = [GroupStep(ps, views[6 + 2 * g], views[7 + 2 * g].view(s_count, max_pages))
                  for g in range(n_groups)]
        max_kv = max(st + q for st, q in zip(starts, q_lens))
        n_single = sum(1 for q in q_lens if q == 1)
        kv_single = max([st + 1 for st, q in zip(starts, q_lens) if q == 1], default=0)
        kv_multi = max([st + q for st, q in zip(starts, q_lens) if q != 1], default=0)
        if pad_pages is not None:
            kv_single = max(kv_single, pad_pages * ps) if n_single else 0
        return StepContext(
            n_tokens=n, n_seqs=s_count, token_ids=views[0], positions=views[1], token_seq=views[2],
            cu_tokens=views[3], state_slots=views[4], want_rows=views[5], groups=groups,
            q_lens=q_lens, kv_starts=starts, state_slots_host=[int(x) for x in state_slots],
            max_q_len=max(q_lens), max_kv_len=max_kv if pad_pages is None else max(max_kv, pad_pages * ps),
            n_single=n_single, max_kv_single=kv_single, max_kv_multi=kv_multi)
