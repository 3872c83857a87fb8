"""Trace replay: given token ids go through the engine's step function one step at a time and
the logits at the wanted places are written out.  Nothing is sampled.

The reference has nothing like it; its closest relative is `bench_generate`, which feeds a
fixed token through prefill and decode (`inferrs/src/engine.rs:2557-2641`).  A trace is a
sequence of JSON objects, one a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step are one batch.  `want` lists places among an entry's tokens whose
logits are written to `<out>/<step>.f32` as little-endian float32 `[wanted, vocab]`, in the
order of the entries and of `want`.  Requests named in `end` give back what they hold after
the step.  After each step `done <step>` is written to `reply` and flushed.
"""
from __future__ import annotations

import json
import os
from typing import IO, Iterable

from .engine import Engine, Entry


class TraceError(ValueError):
    pass


def parse_step(line: str):
    try:
        rec = json.loads(line)
    except json.JSONDecodeError as e:
        raise TraceError(f"a trace line is not valid JSON: {e}") from e
    if not isinstance(rec, dict) or "step" not in rec:
        raise TraceError("a trace line must be an object with a 'step'")
    entries = []
    for e in rec.get("entries") or []:
        if "id" not in e or "tokens" not in e:
            raise TraceError(f"step {rec['step']}: an entry needs 'id' and 'tokens'")
        tokens, want = [int(t) for t in e["tokens"]], [int(w) for w in e.get("want") or []]
        if not tokens and not want:
            continue                                    # (an entry that brings nothing and asks for nothing)
        entries.append(Entry(e["id"], tokens, want))
    return rec["step"], entries, list(rec.get("end") or [])


def run_trace(engine: Engine, lines: Iterable[str], out_dir: str, reply: IO[str]) -> int:
    """Replays `lines`; returns the number of steps run."""
    os.makedirs(out_dir, exist_ok=True)
    steps = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step, entries, end = parse_step(line)
        if entries:
            logits = engine.step(entries)
            if logits.shape[0]:
                logits.cpu().numpy().astype("<f4", copy=False).tofile(os.path.join(out_dir, f"{step}.f32"))
        for seq_id in end:
            if engine.has_request(seq_id):
                engine.end_request(seq_id)
        reply.write(f"done {step}\n")
        reply.flush()
        steps += 1
    return steps
