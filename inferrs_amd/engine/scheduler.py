"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.  Host-only bookkeeping over a `CacheManager`, done by the native runtime; it
never touches the GPU, so its decisions can be tested without one.

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

import ctypes
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

from .. import native
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
    logprobs: List[object] = field(default_factory=list)   # a TokenLogprob per output token, when asked for

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
    """The decisions are taken by the native scheduler (`csrc/runtime.cpp`), which works on the
    cache manager's native object directly; this class names the requests, keeps their Python
    records (`Request`: sampling parameters, seed, output) in step with it and hands out plans."""

    def __init__(self, cache: CacheManager, *, max_batch_size: int = 32, max_tokens_per_step: int = 2048,
                 prefill_chunk: Optional[int] = None, max_seq_len: int = 40960,
                 stop_token_ids: Sequence[int] = (), row_multiple: int = 256):
        """`max_batch_size`: most running requests (the reference's flag of that name, default 32,
        `inferrs/src/main.rs:137-138`); `max_tokens_per_step`: token budget of one step (default
        2048, `main.rs:141-142`); `prefill_chunk`: longest portion of one prompt in a step (None: the
        budget); `max_seq_len`: prompt plus output never exceed it (`inferrs/src/server.rs:3680-3695`);
        `row_multiple`: a portion that is cut (one that does not end its prompt) is cut so that the step's
        tokens, decodes included, are a whole multiple of this, when the step has that many (0 or 1: off).
        The large products walk a step's rows in tiles: 8 decoded tokens beside a portion of 512 cost a layer
        of an 8 B model 250 us in products, beside a portion of 504 212 us."""
        if prefill_chunk is not None and prefill_chunk < 1:
            raise ValueError("prefill_chunk must be >= 1")
        if row_multiple < 0:
            raise ValueError("row_multiple must be >= 0")
        self.cache = cache
        self.max_batch_size = max_batch_size
        self.max_tokens_per_step = max_tokens_per_step
        self.prefill_chunk = prefill_chunk or max_tokens_per_step
        self.max_seq_len = max_seq_len
        self.stop_token_ids = frozenset(int(t) for t in stop_token_ids)
        self._lib = native.runtime()
        stops = sorted(self.stop_token_ids)
        self._ptr = self._lib.iar_sched_create(cache.handle, max_batch_size, max_tokens_per_step, self.prefill_chunk,
                                               max_seq_len, native.ints(stops), len(stops))
        if not self._ptr:
            raise ValueError(native.last_error())
        self.row_multiple = row_multiple
        if self._lib.iar_sched_set_row_multiple(self._ptr, row_multiple) != 0:
            raise ValueError(native.last_error())
        self._requests: Dict[int, Request] = {}      # key -> record of every request not yet finished
        self.finished: Dict[Hashable, Request] = {}
        self._arrivals = 0
        self._room = 0
        self._grow(max(64, max_batch_size))

    def __del__(self):
        if getattr(self, "_ptr", None):
            self._lib.iar_sched_destroy(self._ptr)
            self._ptr = None

    def _grow(self, n: int) -> None:
        """Buffers that the native side fills with up to n requests."""
        if n <= self._room:
            return
        self._room = n
        self._keys = (ctypes.c_int64 * n)()
        self._a, self._b, self._c = (ctypes.c_int * n)(), (ctypes.c_int * n)(), (ctypes.c_int * n)()

    # ---- requests ---------------------------------------------------------------------------
    def add(self, request: Request) -> None:
        key = self.cache.names.pin(request.request_id)
        p = request.params
        extra = [int(t) for t in p.extra_stop_token_ids]
        if self._lib.iar_sched_add(self._ptr, key, native.ints(request.prompt), len(request.prompt), int(p.max_tokens),
                                   int(bool(p.bypass_stop_tokens)), native.ints(extra), len(extra)):
            self.cache.names.unpin(request.request_id, live=request.request_id in self.cache.sequences)
            raise ValueError(f"request {request.request_id!r}: {native.last_error()}")
        request.arrival = self._arrivals
        self._arrivals += 1
        request.status = WAITING
        self._requests[key] = request
        self._grow(len(self._requests))

    def adopt(self, request: Request) -> None:
        """A request that already has a cache entry joins the running requests: its prompt and the
        output so far are given, `computed` becomes what the cache holds of them (their keys and
        values were put there by other means, e.g. a benchmark that fills a context)."""
        name = request.request_id
        if name not in self.cache.sequences:
            raise ValueError(f"request {name!r} has no cache entry")
        key = self.cache.names.pin(name)
        p = request.params
        extra = [int(t) for t in p.extra_stop_token_ids]
        tokens = request.tokens
        got = self._lib.iar_sched_adopt(self._ptr, key, native.ints(tokens), len(tokens), len(request.prompt),
                                        int(p.max_tokens), int(bool(p.bypass_stop_tokens)), native.ints(extra), len(extra))
        if got < 0:
            self.cache.names.unpin(name, live=True)
            raise ValueError(f"request {name!r}: {native.last_error()}")
        request.arrival = self._arrivals
        self._arrivals += 1
        request.status, request.computed = RUNNING, got
        self._requests[key] = request
        self._grow(len(self._requests))

    def has_work(self) -> bool:
        return bool(self._lib.iar_sched_num_waiting(self._ptr) or self._lib.iar_sched_num_running(self._ptr))

    @property
    def waiting(self) -> List[Request]:
        """The line of requests that wait, first in line first."""
        n = self._lib.iar_sched_waiting(self._ptr, self._keys, self._room)
        return [self._requests[k] for k in self._keys[:n]]

    @property
    def running(self) -> List[Request]:
        """The running requests in order of admission."""
        n = self._lib.iar_sched_running(self._ptr, self._keys, self._room)
        return [self._requests[k] for k in self._keys[:n]]

    def _finish(self, key: int, r: Request, reason: str, error: Optional[str] = None) -> None:
        r.status, r.finish_reason, r.error = FINISHED, reason, error
        self.finished[r.request_id] = r
        del self._requests[key]
        self._lib.iar_sched_forget(self._ptr, key)
        self.cache.names.unpin(r.request_id, live=False)

    def finish(self, request: Request, reason: str) -> None:
        """End a waiting or running request now, with `reason` ("stop" when a stop string matched,
        "cancelled" when nobody waits for it any more): what it holds is given back."""
        key = self.cache.names.find(request.request_id)
        if key is None or key not in self._requests:
            return                                      # finished already
        if self._lib.iar_sched_finish(self._ptr, key):
            raise RuntimeError(native.last_error())
        self._finish(key, request, reason)

    # ---- planning ---------------------------------------------------------------------------
    def plan(self) -> Plan:
        """Decide the next step and reserve its pages.  May preempt or fail requests."""
        lib, ptr = self._lib, self._ptr
        plan = Plan()
        n = lib.iar_sched_plan(ptr)
        if n < 0:
            raise RuntimeError(native.last_error())
        for k in self._keys[:lib.iar_sched_plan_preempted(ptr, self._keys, self._room)]:
            r = self._requests[k]
            r.computed, r.status = 0, WAITING
            r.preemptions += 1
            plan.preempted.append(r)
        for k in list(self._keys[:lib.iar_sched_plan_failed(ptr, self._keys, self._room)]):
            r = self._requests[k]
            self._finish(k, r, "error", lib.iar_sched_failure(ptr, k).decode("utf-8", "replace"))
            plan.failed.append(r)
        lib.iar_sched_plan_entries(ptr, self._keys, self._a, self._b, self._c)
        for i in range(n):
            r = self._requests[self._keys[i]]
            r.status = RUNNING
            start, count = self._a[i], self._b[i]
            if count == 1 and start >= len(r.prompt):
                tokens = [r.output[start - len(r.prompt)]]
            else:
                tokens = r.tokens[start:start + count]
            plan.entries.append(PlannedEntry(r, tokens, bool(self._c[i])))
        return plan

    # ---- after the step ---------------------------------------------------------------------
    def _advance(self, finished: int) -> List[Request]:
        done = []
        for k, reason in zip(list(self._keys[:finished]), list(self._a[:finished])):
            r = self._requests[k]
            self._finish(k, r, "stop" if reason == 0 else "length")
            done.append(r)
        return done

    def commit(self, plan: Plan, sampled: Dict[Hashable, int]) -> List[Request]:
        """The step of the latest plan ran: `sampled[request_id]` is the token drawn for every entry
        that `samples`.  Returns the requests that finished."""
        drawn = []
        for e in plan.entries:
            r = e.request
            r.computed += len(e.tokens)
            if e.samples:
                token = int(sampled[r.request_id])
                r.output.append(token)
                drawn.append(token)
        n = self._lib.iar_sched_commit(self._ptr, native.ints(drawn), len(drawn), self._keys, self._a, self._room)
        if n < 0:
            raise RuntimeError(native.last_error())
        return self._advance(n)

    def commit_decode(self, requests: Sequence[Request], tokens: Sequence[int]) -> List[Request]:
        """One decode step of a run that was queued at once: one token for each of `requests` that
        still runs (those that finished earlier in the run are passed over)."""
        keys, toks = [], []
        for r, t in zip(requests, tokens):
            if r.status != RUNNING:
                continue
            r.computed += 1
            r.output.append(int(t))
            keys.append(self.cache.names.find(r.request_id))
            toks.append(int(t))
        n = self._lib.iar_sched_commit_decode(self._ptr, len(keys), native.keys(keys), native.ints(toks),
                                              self._keys, self._a, self._room)
        if n < 0:
            raise RuntimeError(native.last_error())
        return self._advance(n)
