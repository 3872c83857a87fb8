"""The scheduler's decisions, without a GPU: a stand-in executor commits what the scheduler
planned and "samples" a function of the request alone."""
import random

import pytest

from inferrs_amd.cache import CacheManager
from inferrs_amd.engine.scheduler import OUT_OF_BLOCKS, Request, Scheduler
from inferrs_amd.parts.base import PagedKV
from inferrs_amd.sampling import SamplingParams


def make(num_pages=64, page_size=4, max_seqs=8, **kw):
    cache = CacheManager({0: PagedKV(2, 16)}, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs)
    kw.setdefault("max_batch_size", max_seqs)
    return cache, Scheduler(cache, **kw)


def token_for(r):
    """What the stand-in model "generates": depends on the request and its length only."""
    return (hash((r.request_id, r.total)) % 97) + 3


def run(sched, cache, max_steps=10000, trace=None):
    steps = 0
    while sched.has_work():
        plan = sched.plan()
        assert plan.n_tokens <= sched.max_tokens_per_step
        assert len({id(e.request) for e in plan.entries}) == len(plan.entries)
        for e in plan.entries:
            assert e.tokens == e.request.tokens[e.request.computed:e.request.computed + len(e.tokens)]
            assert cache.sequences[e.request.request_id].reserved >= len(e.tokens)
            assert e.samples == (e.request.computed + len(e.tokens) == e.request.total)
        if trace is not None:
            trace.append(plan)
        sched.commit(plan, {e.request.request_id: token_for(e.request) for e in plan.entries if e.samples})
        cache.check_invariants()
        steps += 1
        assert steps < max_steps, "the scheduler does not come to an end"
    return steps


def req(i, n_prompt, max_tokens=8, **kw):
    return Request(i, list(range(1, n_prompt + 1)), SamplingParams.greedy(max_tokens=max_tokens, **kw))


def test_decode_first_then_portions_under_the_budget():
    cache, s = make(max_tokens_per_step=16, prefill_chunk=8)
    a, b = req("a", 5, 4), req("b", 30, 4)
    s.add(a); s.add(b)
    trace = []
    run(s, cache, trace=trace)
    first = trace[0]
    assert [(e.request.request_id, len(e.tokens), e.samples) for e in first.entries] == [("a", 5, True), ("b", 8, False)]
    second = trace[1]       # a decodes first (1 token), b's next portion takes up to the chunk
    assert [(e.request.request_id, len(e.tokens)) for e in second.entries] == [("a", 1), ("b", 8)]
    assert a.finish_reason == b.finish_reason == "length" and len(a.output) == len(b.output) == 4
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


def test_stop_tokens_length_and_context_limit():
    cache, s = make(stop_token_ids=[50], max_seq_len=12)
    a = req("a", 4, 100)
    s.add(a)
    plan = s.plan()
    s.commit(plan, {"a": 50})
    assert a.finish_reason == "stop" and a.output == [50]
    b = req("b", 4, 100, bypass_stop_tokens=True)       # like the reference's bench: stop tokens bypassed
    s.add(b)
    while s.has_work():
        plan = s.plan()
        s.commit(plan, {"b": 50})
    assert b.finish_reason == "length" and b.total == 12           # the context limit
    c = Request("c", [1, 2], SamplingParams.greedy(max_tokens=9, extra_stop_token_ids=(7,)))
    s.add(c)
    s.commit(s.plan(), {"c": 7})
    assert c.finish_reason == "stop"
    with pytest.raises(ValueError, match="limit"):
        s.add(req("d", 12))
    with pytest.raises(ValueError, match="empty"):
        s.add(Request("e", [], SamplingParams()))


def test_admission_stops_at_max_batch_size_and_keeps_arrival_order():
    cache, s = make(max_batch_size=2)
    for i in range(4):
        s.add(req(i, 3, 2))
    plan = s.plan()
    assert [e.request.request_id for e in plan.entries] == [0, 1] and len(s.waiting) == 2
    s.commit(plan, {0: 5, 1: 5})
    plan = s.plan()
    assert [e.request.request_id for e in plan.entries] == [0, 1]
    s.commit(plan, {0: 5, 1: 5})                    # both reach max_tokens and leave
    assert [e.request.request_id for e in s.plan().entries] == [2, 3]


def test_pages_run_out_the_latest_request_is_preempted_and_recomputed():
    # 6 pages of 4 tokens.  a (8 tokens) and b (8 tokens) fill 4; both decode; when b needs the
    # 7th page there is none: b, the latest, goes back to the head of the line.
    cache, s = make(num_pages=6, page_size=4, max_tokens_per_step=64)
    a, b = req("a", 8, 12), req("b", 8, 12)
    s.add(a); s.add(b)
    trace = []
    run(s, cache, trace=trace)
    preempted = [r.request_id for p in trace for r in p.preempted]
    assert preempted and set(preempted) == {"b"} and b.preemptions >= 1 and a.preemptions == 0
    assert a.finish_reason == b.finish_reason == "length" and len(a.output) == len(b.output) == 12
    # recomputation feeds prompt and output so far again, and the result is what an undisturbed run gives
    cache2, s2 = make(num_pages=64, page_size=4)
    b2 = req("b", 8, 12)
    s2.add(b2)
    run(s2, cache2)
    assert b2.output == b.output and b2.preemptions == 0
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


def test_a_request_that_can_never_fit_fails_with_the_reference_error():
    cache, s = make(num_pages=3, page_size=4)
    big, small = req("big", 12, 4), req("small", 3, 2)
    s.add(big); s.add(small)
    run(s, cache)
    assert big.finish_reason == "error" and OUT_OF_BLOCKS in big.error
    assert small.finish_reason == "length"
    # one that fits at first and outgrows the whole pool fails when it does
    cache, s = make(num_pages=3, page_size=4)
    grow = req("grow", 10, 10)
    s.add(grow)
    run(s, cache)
    assert grow.finish_reason == "error" and OUT_OF_BLOCKS in grow.error and len(grow.output) == 3
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


@pytest.mark.parametrize("seed", range(6))
def test_every_request_finishes_whatever_the_order_and_the_pool(seed):
    rng = random.Random(seed)
    page = rng.choice([1, 4, 16])
    cache, s = make(num_pages=rng.randint(40, 120) // page + 8, page_size=page, max_seqs=6,
                    max_batch_size=rng.randint(1, 6), max_tokens_per_step=rng.choice([4, 16, 64]),
                    prefill_chunk=rng.choice([None, 3, 16]))
    reqs = [req(i, rng.randint(1, 30), rng.randint(1, 12)) for i in range(25)]
    pending = list(reqs)
    steps = 0
    while pending or s.has_work():
        for _ in range(rng.randint(0, 3)):
            if pending:
                s.add(pending.pop(0))
        if s.has_work():
            plan = s.plan()
            assert plan.n_tokens <= s.max_tokens_per_step and len(s.running) <= s.max_batch_size
            s.commit(plan, {e.request.request_id: token_for(e.request) for e in plan.entries if e.samples})
            cache.check_invariants()
        steps += 1
        assert steps < 20000
    for r in reqs:
        assert r.finish_reason == "length" and len(r.output) == r.params.max_tokens, (r.request_id, r.finish_reason, r.error)
        # outputs do not depend on interleaving or preemption: each token is a function of the request alone
        alone = Request(r.request_id, list(r.prompt), r.params)
        while len(alone.output) < r.params.max_tokens:
            alone.output.append(token_for(alone))
        assert alone.output == r.output
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups) and cache.slots.num_free == 6


def test_a_request_with_a_cache_entry_can_be_adopted():
    cache, s = make(num_pages=16, page_size=4)
    cache.add_sequence("a")
    assert cache.reserve("a", 10)
    cache.commit("a", 10)
    a = Request("a", list(range(10)), SamplingParams.greedy(max_tokens=3), output=[77])
    s.adopt(a)
    assert a.status == "running" and a.computed == 10 and [r.request_id for r in s.running] == ["a"]
    plan = s.plan()
    assert [(e.request.request_id, e.tokens, e.samples) for e in plan.entries] == [("a", [77], True)]
    assert s.commit(plan, {"a": 5}) == [] and a.output == [77, 5]
    run(s, cache)
    assert a.finish_reason == "length" and len(a.output) == 3
    assert cache.groups[0].pool.num_free == 16 and not cache.names.names()
    with pytest.raises(ValueError, match="no cache entry"):
        s.adopt(Request("b", [1, 2], SamplingParams.greedy()))
    cache.add_sequence("c")
    assert cache.reserve("c", 2)
    cache.commit("c", 2)
    with pytest.raises(ValueError, match="at least one must be left"):
        s.adopt(Request("c", [1, 2], SamplingParams.greedy()))


def test_a_name_in_use_outside_the_scheduler_is_reported():
    cache, s = make()
    cache.add_sequence("a")                        # somebody else's request of the same name
    s.add(req("a", 3))
    with pytest.raises(RuntimeError, match="already live"):
        s.plan()


def test_a_request_can_be_ended_from_outside():
    cache, s = make(num_pages=16, page_size=4, max_tokens_per_step=8)
    a, b, c = req("a", 6, 10), req("b", 20, 10), req("c", 3, 10)
    for r in (a, b, c):
        s.add(r)
    plan = s.plan()                                  # a whole, the first two tokens of b
    assert [(e.request.request_id, len(e.tokens)) for e in plan.entries] == [("a", 6), ("b", 2)]
    s.finish(b, "cancelled")                         # while its portion is planned
    assert b.finish_reason == "cancelled" and "b" not in cache.sequences
    s.finish(c, "cancelled")                         # while it waits
    assert c.status == "finished" and [r.request_id for r in s.waiting] == []
    s.finish(c, "cancelled")                         # again: nothing happens
    run(s, cache)
    assert a.finish_reason == "length" and len(a.output) == 10
    assert cache.groups[0].pool.num_free == 16 and not cache.names.names()


def test_a_budget_below_the_number_of_decodes_starves_nobody():
    """Five requests decode under a budget of two tokens a step: those left out of a step go first in
    the next, so that every request advances at the same pace (two steps out of five)."""
    cache, s = make(max_tokens_per_step=2, max_seqs=5)
    reqs = [req(i, 2, max_tokens=6) for i in range(5)]
    for r in reqs:
        s.add(r)
    trace = []
    run(s, cache, trace=trace)
    assert all(r.finish_reason == "length" and len(r.output) == 6 for r in reqs)
    decodes = [[e.request.request_id for e in p.entries if len(e.tokens) == 1 and e.request.output] for p in trace]
    served = {i: [k for k, ids in enumerate(decodes) if i in ids] for i in range(5)}
    # nobody waits more than three steps between two of its decodes while all five are decoding
    both = [k for k, ids in enumerate(decodes) if len(ids) == 2]
    for i in range(5):
        gaps = [b - a for a, b in zip(served[i], served[i][1:]) if a in both and b in both]
        assert gaps and max(gaps) <= 3, (i, served[i])


def test_make_trace_program_and_modes(tmp_path):
    """`bin/make_trace` and `make_trace`: every mode feeds every token of every request exactly once and in order,
    asks for every position's logits once, ends every request, and states the pool that the replay needs."""
    import json
    import os
    import subprocess
    import sys
    from inferrs_amd.engine.trace import MODES, make_trace
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    requests = {"a": list(range(3)), "b": list(range(100, 170)), "c": list(range(200, 333)), "d": [7]}
    for mode in MODES:
        trace = make_trace(requests, mode, tail=9, sizes=[5, 2, 31], seed=3, max_live=3)
        fed = {r: [] for r in requests}
        wanted = {r: [] for r in requests}
        ended = []
        for i, line in enumerate(trace.lines):
            rec = json.loads(line)
            assert rec["step"] == i
            for e in rec["entries"]:
                assert e["id"] not in ended
                start = len(fed[e["id"]])
                fed[e["id"]] += e["tokens"]
                wanted[e["id"]] += [start + w for w in e["want"]]
            ended += rec["end"]
        assert fed == requests and sorted(ended) == sorted(requests), mode
        assert all(wanted[r] == list(range(len(t))) for r, t in requests.items()), mode
        assert trace.max_live <= (3 if mode == "mixed" else 1)
        assert trace.max_tokens >= 192 and trace.max_tokens % 64 == 0
    with pytest.raises(ValueError, match="unknown mode"):
        make_trace(requests, "sideways")
    manifest = tmp_path / "m.json"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "make_trace"), "--mode", "mixed", "--lengths", "5,37,70",
                           "--vocab", "50", "--seed", "4", "--manifest", str(manifest)], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    info = json.loads(manifest.read_text())
    lines = proc.stdout.splitlines()
    assert sorted(len(t) for t in info["requests"].values()) == [5, 37, 70] and info["max_tokens"] % 64 == 0
    assert sum(len(rows) for rows in info["rows"].values()) == 112 and len(lines) > 10
    assert all(0 <= t < 50 for line in lines for e in json.loads(line)["entries"] for t in e["tokens"])


def test_cut_portions_make_the_steps_rows_a_whole_multiple():
    """With `row_multiple` a portion that does not end its prompt is cut so that the step's tokens (decodes first, then
    portions) are a whole multiple of it; a portion that ends its prompt is left alone, and so are steps with fewer
    tokens than one multiple."""
    cache = CacheManager({0: PagedKV(2, 16)}, 16, 400, 8)
    sched = Scheduler(cache, max_batch_size=8, max_tokens_per_step=96, prefill_chunk=40, row_multiple=32)
    long = Request("long", list(range(1, 131)), SamplingParams.greedy(max_tokens=4))
    sched.add(long)
    plan = sched.plan()
    assert [len(e.tokens) for e in plan.entries] == [32]              # 40 would leave 8 over a multiple
    sched.commit(plan, {})
    short = Request("short", [5, 6, 7], SamplingParams.greedy(max_tokens=6))
    sched.add(short)
    plan = sched.plan()
    # the running request's portion first (32 again), then the newcomer's whole prompt, which ends it: 35 tokens
    assert [(e.request.request_id, len(e.tokens), e.samples) for e in plan.entries] == [("long", 32, False), ("short", 3, True)]
    sched.commit(plan, {"short": 9})
    plan = sched.plan()
    # one decode, then a portion cut to 31 so that the step has 32 tokens
    assert [(e.request.request_id, len(e.tokens)) for e in plan.entries] == [("short", 1), ("long", 31)]
    sched.commit(plan, {"short": 9})
    plan = sched.plan()
    # 35 tokens are left of the long prompt: they end it and are taken whole
    assert [(e.request.request_id, len(e.tokens), e.samples) for e in plan.entries] == [("short", 1, True), ("long", 35, True)]
    # switched off, the portions are the chunk
    off = Scheduler(CacheManager({0: PagedKV(2, 16)}, 16, 400, 8), max_batch_size=8, max_tokens_per_step=96, prefill_chunk=40,
                    row_multiple=0)
    off.add(Request("long", list(range(1, 131)), SamplingParams.greedy(max_tokens=4)))
    assert [len(e.tokens) for e in off.plan().entries] == [40]
    with pytest.raises(ValueError, match="row_multiple"):
        Scheduler(cache, max_batch_size=8, row_multiple=-1)


def test_a_trace_line_is_read_as_it_is_written():
    """The replay's reader: entries in their order with their wanted places in theirs, ids of any JSON kind, an entry that
    brings nothing and asks for nothing left out, a step of nothing but ends, and errors that say what is missing."""
    from inferrs_amd.engine.replay import TraceError, parse_step
    step, entries, end = parse_step('{"step": 7, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [2, 0]}, '
                                    '{"id": 4, "tokens": [9]}, {"id": "c", "tokens": [], "want": []}], "end": ["a"]}')
    assert step == 7 and end == ["a"]
    assert [(e.seq_id, e.tokens, e.want) for e in entries] == [("a", [5, 17, 3], [2, 0]), (4, [9], [])]
    assert parse_step('{"step": 8, "end": ["b"]}') == (8, [], ["b"])
    assert parse_step('{"step": 9, "entries": null, "end": null}') == (9, [], [])
    for bad in ('{"entries": []}', 'not json', '[1, 2]', '{"step": 1, "entries": [{"tokens": [1]}]}',
                '{"step": 1, "entries": [{"id": "a"}]}'):
        with pytest.raises(TraceError):
            parse_step(bad)
