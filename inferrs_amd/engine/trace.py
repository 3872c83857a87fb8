"""Builders of replay traces for the ways a request's tokens may be cut into steps, and the
reader of what a replay wrote (the companion of `inferrs_amd.engine.replay` and `bin/trace_run`;
`bin/make_trace` is its command line).  The reference has nothing like it.

A `Trace` records, for every step with wanted logits, which (request, position) each row belongs
to, and how many cache tokens the live requests hold at most (each rounded up to 64), which is what
the replay's pool is made for.  The modes: `whole` (each request alone, all tokens in one step),
`prefix_then_single` (all but a tail in one step, then token by token), `portions` (alone, in
portions of changing size) and `mixed` (several live requests, portions of some beside single
tokens of others, finished requests' pages used again)."""
from __future__ import annotations

import json
import os
import random
from typing import Dict, List, Sequence, Tuple

import numpy as np


def round_up(n: int, m: int) -> int:
    return -(-n // m) * m


class Trace:
    def __init__(self):
        self.lines: List[str] = []
        self.rows: Dict[int, List[Tuple[str, int]]] = {}     # step -> [(request, position)]
        self.fed: Dict[str, int] = {}                        # live request -> tokens fed so far
        self.max_tokens = 0
        self.max_live = 0

    def step(self, entries: Sequence[Tuple[str, Sequence[int], Sequence[int]]], end: Sequence[str] = ()):
        """entries: (request, its next tokens, wanted places among them)."""
        n = len(self.lines)
        rows = []
        for rid, toks, want in entries:
            start = self.fed.get(rid, 0)
            rows += [(rid, start + w) for w in want]
            self.fed[rid] = start + len(toks)
        self.max_tokens = max(self.max_tokens, sum(round_up(v, 64) for v in self.fed.values()))
        self.max_live = max(self.max_live, len(self.fed))
        if rows:
            self.rows[n] = rows
        self.lines.append(json.dumps({
            "step": n, "entries": [{"id": r, "tokens": list(map(int, t)), "want": list(map(int, w))}
                                   for r, t, w in entries], "end": list(end)}))
        for rid in end:
            del self.fed[rid]

    def text(self) -> str:
        return "".join(l + "\n" for l in self.lines)

    def read(self, out_dir: str, vocab: int) -> Dict[str, Dict[int, np.ndarray]]:
        """request -> position -> logits row, from the files a replay wrote."""
        got: Dict[str, Dict[int, np.ndarray]] = {}
        for step, rows in self.rows.items():
            arr = np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4")
            assert arr.size == len(rows) * vocab, f"step {step}: {arr.size} floats for {len(rows)} rows of {vocab}"
            arr = arr.reshape(len(rows), vocab)
            for (rid, pos), row in zip(rows, arr):
                assert pos not in got.setdefault(rid, {}), f"{rid}: position {pos} written twice"
                got[rid][pos] = row
        return got


def whole(requests: Dict[str, List[int]]) -> Trace:
    """Each request alone, all its tokens in one step."""
    t = Trace()
    for rid, toks in requests.items():
        t.step([(rid, toks, range(len(toks)))], end=[rid])
    return t


def prefix_then_single(requests: Dict[str, List[int]], tail: int = 32) -> Trace:
    """All but the last `tail` tokens in one step, then one token a step."""
    t = Trace()
    for rid, toks in requests.items():
        cut = max(1, len(toks) - tail)
        t.step([(rid, toks[:cut], range(cut))])
        for i in range(cut, len(toks)):
            t.step([(rid, toks[i:i + 1], [0])], end=[rid] if i == len(toks) - 1 else [])
        if cut == len(toks):
            t.step([], end=[rid])
    return t


def portions(requests: Dict[str, List[int]], sizes: Sequence[int]) -> Trace:
    """Each request alone, in portions whose sizes cycle through `sizes` (down to two tokens)."""
    t = Trace()
    for rid, toks in requests.items():
        i = k = 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            t.step([(rid, toks[i:i + n], range(n))], end=[rid] if i + n == len(toks) else [])
            i += n
    return t


def mixed(requests: Dict[str, List[int]], seed: int, max_live: int = 4, decode_tail: int = 24,
          sizes: Sequence[int] = (2, 3, 5, 7, 16, 31, 64)) -> Trace:
    """Up to `max_live` requests at a time: portions of some prompts beside single decoded
    tokens of others; a request is sometimes left out of a step; a finished request's pages
    go back and the next request starts."""
    rng = random.Random(seed)
    t = Trace()
    waiting = list(requests)
    live: List[str] = []
    pos = {r: 0 for r in requests}
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            live.append(waiting.pop(0))
        entries, end = [], []
        for rid in list(live):
            toks = requests[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                        # sits this step out
            left = len(toks) - pos[rid]
            n = 1 if left <= decode_tail else min(rng.choice(sizes), left - decode_tail)
            entries.append((rid, toks[pos[rid]:pos[rid] + n], range(n)))
            pos[rid] += n
            if pos[rid] == len(toks):
                end.append(rid)
                live.remove(rid)
        if entries:
            t.step(entries, end=end)
    return t


MODES = ("whole", "tail", "portions", "mixed")


def make_trace(requests: Dict[str, List[int]], mode: str, *, tail: int = 32, sizes: Sequence[int] = (7, 2, 16, 3, 2, 33, 5, 2, 64),
               seed: int = 0, max_live: int = 4) -> Trace:
    """The trace of `requests` (name -> token ids) in one of `MODES`.  `tail`: tokens fed one by one at the end
    ("tail", and in "mixed" the stretch of a request that is decoded); `sizes`: the portions' sizes, cycled
    ("portions"); `seed`, `max_live`: the random interleaving and the most live requests ("mixed")."""
    if mode == "whole":
        return whole(requests)
    if mode == "tail":
        return prefix_then_single(requests, tail)
    if mode == "portions":
        return portions(requests, sizes)
    if mode == "mixed":
        return mixed(requests, seed, max_live=max_live, decode_tail=tail)
    raise ValueError(f"unknown mode {mode!r}; one of {MODES}")
