"""A plain Python cache manager and scheduler: the oracle that the native runtime
(`inferrs_amd/csrc/runtime.cpp`) is compared with, decision for decision, under random orders of
requests.  It shares no code with the product: needs are told apart by their attributes
(`window` for pages, `shape` for state), requests are this file's own records.

Rules written down here: pages are addressed as in the reference's `BlockPool` / `BlockTable`
(`inferrs-models/src/kv_cache.rs:80-140`, `:154-222`), free pages form a FIFO; a request stops as
`check_stop` says (`inferrs/src/engine.rs:866-887`); out of pages is the reference's "paged
attention: out of KV blocks" (`engine.rs:2093-2095`)."""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

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
    need: object
    layers: List[int]
    pool: PagePool


@dataclass
class StateInfo:
    layer: int
    need: object


@dataclass
class SequenceCache:
    seq_id: Hashable
    length: int = 0                                   # tokens whose keys are cached
    tables: Dict[int, List[int]] = field(default_factory=dict)   # group -> logical page -> physical
    state_slot: int = -1
    reserved: int = 0                                 # tokens reserved beyond `length`


def group_layers(needs: Dict[int, object]):
    """Cache-owning layers -> (paged groups in order of first layer, state layers)."""
    groups: Dict[PagedKV, List[int]] = {}
    states: List[StateInfo] = []
    for layer in sorted(needs):
        need = needs[layer]
        if need is None:
            continue
        if hasattr(need, 'window'):
            groups.setdefault(need, []).append(layer)
        elif hasattr(need, 'shape'):
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


# ---- scheduler -------------------------------------------------------------------------------
WAITING, RUNNING, FINISHED = "waiting", "running", "finished"
OUT_OF_BLOCKS = "paged attention: out of KV blocks"


@dataclass
class Request:
    request_id: Hashable
    prompt: List[int]
    params: object
    seed: int = 0
    output: List[int] = field(default_factory=list)
    computed: int = 0                   # tokens whose keys and values are in the cache
    status: str = WAITING
    finish_reason: Optional[str] = None  # "stop" | "length" | "error"
    error: Optional[str] = None
    preemptions: int = 0
    arrival: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def total(self) -> int:
        return len(self.prompt) + len(self.output)


@dataclass
class PlannedEntry:
    request: Request
    tokens: List[int]
    samples: bool                       # the last of these tokens is the request's last: its logits are wanted


@dataclass
class Plan:
    entries: List[PlannedEntry] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    failed: List[Request] = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)


class Scheduler:
    def __init__(self, cache: CacheManager, *, max_batch_size: int = 32, max_tokens_per_step: int = 2048,
                 prefill_chunk: Optional[int] = None, max_seq_len: int = 40960,
                 stop_token_ids: Sequence[int] = (), row_multiple: int = 256):
        """`max_batch_size`: most running requests (the reference's flag of that name, default 32,
        `inferrs/src/main.rs:137-138`); `max_tokens_per_step`: token budget of one step (default
        2048, `main.rs:141-142`); `prefill_chunk`: longest portion of one prompt in a step (None: the
        budget); `max_seq_len`: prompt plus output never exceed it (`inferrs/src/server.rs:3680-3695`)."""
        if max_batch_size < 1 or max_tokens_per_step < 1:
            raise ValueError("max_batch_size and max_tokens_per_step must be >= 1")
        if max_batch_size > cache.max_seqs:
            raise ValueError(f"max_batch_size {max_batch_size} exceeds the cache's {cache.max_seqs} request slots")
        if prefill_chunk is not None and prefill_chunk < 1:
            raise ValueError("prefill_chunk must be >= 1")
        self.cache = cache
        self.max_batch_size = max_batch_size
        self.max_tokens_per_step = max_tokens_per_step
        self.prefill_chunk = prefill_chunk or max_tokens_per_step
        self.max_seq_len = max_seq_len
        self.row_multiple = row_multiple
        self.stop_token_ids = frozenset(int(t) for t in stop_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []            # in order of admission
        self.finished: Dict[Hashable, Request] = {}
        self._arrivals = 0
        self._left_out: set = set()                 # decodes that found no budget in the last plan

    def _portion(self, left: int, budget: int) -> int:
        """Tokens of a request that this step takes: a portion that does not end its prompt is cut so that the step's
        tokens so far are a whole multiple of `row_multiple`, when the step has that many."""
        n = min(left, self.prefill_chunk, budget)
        if self.row_multiple > 1 and n < left:
            rows = self.max_tokens_per_step - budget + n
            over = rows % self.row_multiple
            if over and rows - over >= self.row_multiple and n - over >= 1:
                n -= over
        return n

    # ---- requests ---------------------------------------------------------------------------
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise ValueError(f"request {request.request_id!r}: the prompt is empty")
        if len(request.prompt) >= self.max_seq_len:
            raise ValueError(f"request {request.request_id!r}: the prompt has {len(request.prompt)} tokens, "
                             f"the limit is {self.max_seq_len - 1}")
        request.arrival = self._arrivals
        self._arrivals += 1
        request.status = WAITING
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _pages_total(self) -> int:
        return min(g.pool.num_pages for g in self.cache.groups) if self.cache.groups else 1 << 60

    def _fits_alone(self, n_tokens: int) -> bool:
        return -(-n_tokens // self.cache.page_size) <= self._pages_total()

    # ---- planning ---------------------------------------------------------------------------
    def plan(self) -> Plan:
        """Decide the next step and reserve its pages.  May preempt or fail requests."""
        plan = Plan()
        budget = self.max_tokens_per_step

        # 1. decodes: running requests with exactly one token left to feed
        decoding = [r for r in self.running if r.total - r.computed == 1 and r.output]
        # whoever was left out for lack of budget last time goes first, then the others (admission order)
        decoding = ([r for r in decoding if r.request_id in self._left_out]
                    + [r for r in decoding if r.request_id not in self._left_out])
        self._left_out = set()
        for r in decoding:
            if r not in self.running:               # preempted while serving an earlier one
                continue
            if budget < 1:
                self._left_out.add(r.request_id)
                continue
            while not self.cache.reserve(r.request_id, 1):
                victim = self._preempt_latest(exclude=r)
                if victim is None:
                    # it holds every page there is and needs one more: it cannot go on
                    self._fail(r, f"{OUT_OF_BLOCKS} at position {r.computed}")
                    plan.failed.append(r)
                    break
                plan.preempted.append(victim)
                budget += sum(len(e.tokens) for e in plan.entries if e.request is victim)
                plan.entries = [e for e in plan.entries if e.request is not victim]
            else:
                plan.entries.append(PlannedEntry(r, [r.tokens[-1]], True))
                budget -= 1

        # 2. portions of prompts of running requests, oldest first
        planned = {id(e.request) for e in plan.entries}
        for r in list(self.running):
            if budget < 1:
                break
            if id(r) in planned or r.total - r.computed < 1:
                continue
            if r.total - r.computed == 1 and r.output:
                continue                                  # a decode that found no budget
            n = self._portion(r.total - r.computed, budget)
            if not self.cache.reserve(r.request_id, n):
                continue                                  # waits for pages; decodes above free them as they finish
            plan.entries.append(PlannedEntry(r, r.tokens[r.computed:r.computed + n], r.computed + n == r.total))
            budget -= n

        # 3. admissions, in arrival order
        while self.waiting and budget >= 1 and len(self.running) < self.max_batch_size:
            r = self.waiting[0]
            if not self._fits_alone(r.total + 1):
                self.waiting.popleft()
                self._fail(r, f"{OUT_OF_BLOCKS}: the request needs {-(-(r.total + 1) // self.cache.page_size)} "
                              f"pages, the pool has {self._pages_total()}", live=False)
                plan.failed.append(r)
                continue
            n = self._portion(r.total - r.computed, budget)
            self.cache.add_sequence(r.request_id)
            # admitted only when all it has so far, and one token more, would fit now: a request
            # that is let in on its first portion alone tends to be preempted later
            if not self.cache.can_reserve([(r.request_id, r.total + 1)]) or not self.cache.reserve(r.request_id, n):
                self.cache.free_sequence(r.request_id)
                break                                     # no pages now: it stays first in line
            self.waiting.popleft()
            r.status = RUNNING
            self.running.append(r)
            plan.entries.append(PlannedEntry(r, r.tokens[r.computed:r.computed + n], r.computed + n == r.total))
            budget -= n

        if not plan.entries and self.running and not plan.failed and not plan.preempted:
            # Every running request waits for pages that nobody will free: preempt the latest so
            # that the oldest can go on.
            victim = self._preempt_latest(exclude=self.running[0])
            if victim is not None:
                plan.preempted.append(victim)
                return self._merge(plan, self.plan())
            r = self.running[0]
            self._fail(r, f"{OUT_OF_BLOCKS} at position {r.computed}")
            plan.failed.append(r)
        return plan

    @staticmethod
    def _merge(first: Plan, second: Plan) -> Plan:
        second.preempted = first.preempted + second.preempted
        second.failed = first.failed + second.failed
        return second

    def _preempt_latest(self, exclude: Request) -> Optional[Request]:
        for victim in reversed(self.running):
            if victim is exclude:
                continue
            self.running.remove(victim)
            self.cache.free_sequence(victim.request_id)
            victim.computed = 0
            victim.status = WAITING
            victim.preemptions += 1
            self.waiting.appendleft(victim)
            return victim
        return None

    def _fail(self, r: Request, message: str, live: bool = True) -> None:
        if live:
            if r in self.running:
                self.running.remove(r)
            if r.request_id in self.cache.sequences:
                self.cache.free_sequence(r.request_id)
        r.status, r.finish_reason, r.error = FINISHED, "error", message
        self.finished[r.request_id] = r

    # ---- after the step ---------------------------------------------------------------------
    def commit(self, plan: Plan, sampled: Dict[Hashable, int]) -> List[Request]:
        """The step ran: `sampled[request_id]` is the token drawn for every entry that
        `samples`.  Returns the requests that finished."""
        done: List[Request] = []
        for e in plan.entries:
            r = e.request
            self.cache.commit(r.request_id, len(e.tokens))
            r.computed += len(e.tokens)
            if not e.samples:
                continue
            token = int(sampled[r.request_id])
            r.output.append(token)
            reason = self._stop_reason(r, token)
            if reason is not None:
                r.status, r.finish_reason = FINISHED, reason
                self.running.remove(r)
                self.cache.free_sequence(r.request_id)
                self.finished[r.request_id] = r
                done.append(r)
        return done

    def _stop_reason(self, r: Request, token: int) -> Optional[str]:
        """`check_stop` of the reference (`inferrs/src/engine.rs:866-887`): a stop token ends with
        "stop" unless stop tokens are bypassed; reaching max_tokens or the context limit with "length"."""
        p = r.params
        if not p.bypass_stop_tokens and (token in self.stop_token_ids or token in p.extra_stop_token_ids):
            return "stop"
        if len(r.output) >= p.max_tokens:
            return "length"
        if r.total >= self.max_seq_len:
            return "length"
        return None
