"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.  Host-only bookkeeping over a `CacheManager`; it never touches the GPU, so
its decisions can be tested without one.

The reference's loop (`inferrs/src/engine.rs:1380-1912`) admits from a FIFO channel while
fewer than `max_batch_size` requests are active, runs each request's whole prompt in one pass
and then one forward per active request per round; `--max-tokens-per-step` is parsed and unused
(`engine.rs:1389`), and a request that finds no free block fails with "paged attention: out of
KV blocks" (`engine.rs:2093-2095`).  Here one step serves all running requests together:

  1. every running request whose tokens are all but one in the cache decodes (one token each);
  2. what is left of the token budget goes to portions of prompts, oldest request first;
  3. waiting requests are admitted in arrival order while fewer than `max_batch_size` run and
     pages for their first portion are free.

A request's tokens are its prompt followed by its output; `computed` of them are in the cache.
Each step feeds the next few, and when the last one has been fed the logits at that place
give the next output token.  That one rule covers prompts, decoding and recomputation.

When pages run out for a decoding request, the most recently admitted running request is
preempted: its pages are freed and it goes back to the head of the waiting line with
`computed = 0`, to be recomputed (prompt and output so far) when pages are free again.  A
request that could not fit even alone fails with the reference's error.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"
OUT_OF_BLOCKS = "paged attention: out of KV blocks"


@dataclass
class Request:
    request_id: Hashable
    prompt: List[int]
    params: SamplingParams
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
                 stop_token_ids: Sequence[int] = ()):
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
        self.stop_token_ids = frozenset(int(t) for t in stop_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []            # in order of admission
        self.finished: Dict[Hashable, Request] = {}
        self._arrivals = 0

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
        for r in decoding:
            if r not in self.running:               # preempted while serving an earlier one
                continue
            if budget < 1:
                break
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
            n = min(r.total - r.computed, self.prefill_chunk, budget)
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
            n = min(r.total - r.computed, self.prefill_chunk, budget)
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
