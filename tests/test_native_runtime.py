"""The native runtime (`inferrs_amd/csrc/runtime.cpp`) against the plain Python one in
`plain_runtime.py`: the same random orders of requests go through both, and every answer, block
table, free count, plan and finish must be the same.  Step assembly is compared with a NumPy
assembly written here.  No GPU is needed."""
import ctypes
import random
from types import SimpleNamespace

import numpy as np
import pytest

import plain_runtime as plain
from inferrs_amd import native
from inferrs_amd.cache import CacheError, CacheManager
from inferrs_amd.engine.scheduler import Request, Scheduler
from inferrs_amd.parts.base import FixedState, PagedKV
from inferrs_amd.sampling import SamplingParams

FULL = PagedKV(2, 16)


def both_caches(rng, windows=True):
    page = rng.choice([1, 3, 4, 16])
    needs = {0: FULL, 1: PagedKV(2, 16, window=rng.choice([5, 10, 33])) if windows else FULL, 2: FULL, 3: FixedState((4,))}
    n_groups = 2 if windows else 1
    pages = [rng.randint(4, 40) for _ in range(n_groups)]
    max_seqs = rng.randint(2, 6)
    return (CacheManager(needs, page, pages, max_seqs), plain.CacheManager(needs, page, pages, max_seqs), page, max_seqs)


def same_state(a, b, live):
    assert len(a.sequences) == len(b.sequences) == len(live)
    assert [g.pool.num_free for g in a.groups] == [g.pool.num_free for g in b.groups]
    assert a.slots.num_free == b.slots.num_free
    for sid in live:
        x, y = a.sequences[sid], b.sequences[sid]
        assert (x.length, x.reserved, x.state_slot) == (y.length, y.reserved, y.state_slot)
        assert x.tables.values() == [y.tables[g] for g in range(len(b.groups))]


@pytest.mark.parametrize("seed", range(10))
def test_cache_manager_gives_the_answers_of_the_plain_one(seed):
    rng = random.Random(seed)
    a, b, page, max_seqs = both_caches(rng)
    live, next_id = [], 0
    for _ in range(1200):
        roll = rng.random()
        if roll < 0.15:
            if len(live) < max_seqs:
                assert a.add_sequence(next_id).state_slot == b.add_sequence(next_id).state_slot
                live.append(next_id)
                next_id += 1
            else:
                with pytest.raises(CacheError, match="slots are in use"):
                    a.add_sequence("one too many")
        elif roll < 0.28 and live:
            sid = live.pop(rng.randrange(len(live)))
            a.free_sequence(sid)
            b.free_sequence(sid)
        elif roll < 0.34 and live:
            asks = [(s, rng.choice([1, 5, 40])) for s in rng.sample(live, rng.randint(1, len(live)))]
            assert a.can_reserve(asks) == b.can_reserve(asks)
        elif live:
            sid = rng.choice(live)
            n = rng.choice([1, 1, 1, 2, 7, 33])
            got = a.reserve(sid, n)
            assert got == b.reserve(sid, n)
            if got:
                k = rng.randint(0, n) if rng.random() < 0.3 else n
                a.commit(sid, k)
                b.commit(sid, k)
                seq = b.sequences[sid]
                start = rng.randint(max(0, seq.length - 3), seq.length)
                for g in range(len(b.groups)):
                    count = min(3, seq.length + seq.reserved - start)
                    try:
                        want = b.slot_ids(sid, g, start, count)
                    except plain.CacheError:
                        with pytest.raises(CacheError, match="released"):
                            a.slot_ids(sid, g, start, count)
                    else:
                        assert a.slot_ids(sid, g, start, count) == want
        same_state(a, b, live)
        a.check_invariants()
    with pytest.raises(CacheError, match="commit"):
        if not live:
            live.append(next_id)
            a.add_sequence(next_id)
        a.commit(live[0], a.sequences[live[0]].reserved + 1)


def test_batchwise_calls_top_up_for_all_or_for_none():
    m = CacheManager({0: FULL}, page_size=4, num_pages=5, max_seqs=3)
    for s in "abc":
        m.add_sequence(s)
    assert m.all_live(["a", "b", "c"]) and not m.all_live(["a", "z"])
    assert m.reserve("a", 6)                                             # 2 pages
    assert m.ensure_reserved([("a", 8), ("b", 4), ("c", 1)])            # a: nothing new (8 fit its 2 pages), b 1, c 1
    assert [m.sequences[s].reserved for s in "abc"] == [8, 4, 1] and m.groups[0].pool.num_free == 1
    assert not m.ensure_reserved([("b", 8), ("c", 8)])                   # 2 pages wanted, 1 free: nothing is taken
    assert [m.sequences[s].reserved for s in "abc"] == [8, 4, 1] and m.groups[0].pool.num_free == 1
    m.commit_many([("a", 8), ("b", 2)])
    assert m.max_length(["a", "b", "c"]) == 8 and m.max_length(["b", "c"]) == 2
    with pytest.raises(CacheError, match="not live"):
        m.max_length(["a", "nobody"])
    m.check_invariants()


# ---- step assembly ----------------------------------------------------------------------------
def plain_step(cache: plain.CacheManager, entries, pad_pages, advance):
    """The arrays of one step, from the plain cache manager: single-token requests first."""
    ps = cache.page_size
    order = sorted(range(len(entries)), key=lambda i: len(entries[i][1]) != 1)
    rank = {orig: new for new, orig in enumerate(order)}
    ordered = [entries[i] for i in order]
    seqs = [cache.sequences[e[0]] for e in ordered]
    q = [len(e[1]) for e in ordered]
    starts = [s.length + advance for s in seqs]
    cu = np.concatenate([[0], np.cumsum(q)]).astype(np.int32)
    max_pages = max(1, max(-(-(st + n) // ps) for st, n in zip(starts, q)))
    if pad_pages:
        max_pages = pad_pages
    out = [np.concatenate([np.asarray(e[1], dtype=np.int32) for e in ordered]),
           np.concatenate([np.arange(st, st + n, dtype=np.int32) for st, n in zip(starts, q)]),
           np.repeat(np.arange(len(q), dtype=np.int32), q), cu,
           np.asarray([s.state_slot for s in seqs], dtype=np.int32),
           np.asarray([cu[rank[i]] + w for i, e in enumerate(entries) for w in e[2]], dtype=np.int32)]
    for g in range(len(cache.groups)):
        table = np.zeros((len(q), max_pages), dtype=np.int32)
        slots = []
        for i, s in enumerate(seqs):
            row = s.tables[g]
            table[i, :min(len(row), max_pages)] = [max(p, 0) for p in row[:max_pages]]
            slots += cache.slot_ids(s.seq_id, g, starts[i], q[i])
        out += [np.asarray(slots, dtype=np.int32), table.reshape(-1)]
    kv = [st + n for st, n in zip(starts, q)]
    singles = [k for k, n in zip(kv, q) if n == 1]
    multis = [k for k, n in zip(kv, q) if n != 1]
    meta = dict(n=sum(q), max_pages=max_pages, max_q=max(q), n_single=len(singles),
                max_kv=max(kv + ([pad_pages * ps] if pad_pages else [])),
                kv_single=max(singles + ([pad_pages * ps] if pad_pages and singles else []), default=0),
                kv_multi=max(multis + ([pad_pages * ps] if pad_pages and multis else []), default=0))
    return np.concatenate(out), meta, order


def native_step(cache: CacheManager, entries, pad_pages, advance):
    lib = native.runtime()
    ks = native.keys([cache.names.find(e[0]) for e in entries])
    q = native.ints([len(e[1]) for e in entries])
    tokens = native.ints([t for e in entries for t in e[1]])
    wc = native.ints([len(e[2]) for e in entries])
    want = native.ints([w for e in entries for w in e[2]])
    words = lib.iar_step_words(cache.handle, len(entries), ks, q, len(want), pad_pages, advance)
    assert words >= 0, native.last_error()
    out = np.full(words + 8, -7, dtype=np.int32)
    meta, order = (ctypes.c_int * 16)(), (ctypes.c_int * len(entries))()
    code = lib.iar_build_step(cache.handle, len(entries), ks, q, ctypes.addressof(tokens), wc, want, pad_pages,
                              advance, out.ctypes.data, words, meta, order)
    if code:
        raise ValueError(native.last_error())
    assert meta[0] == words and (out[words:] == -7).all()          # exactly the announced words are written
    return out[:words], meta, list(order)


@pytest.mark.parametrize("seed", range(8))
def test_step_assembly_matches_a_numpy_assembly(seed):
    rng = random.Random(100 + seed)
    a, b, page, max_seqs = both_caches(rng)
    live = []
    for sid in range(max_seqs):
        n = rng.randint(0, 50)
        a.add_sequence(sid); b.add_sequence(sid)
        if a.reserve(sid, n):
            assert b.reserve(sid, n)
            a.commit(sid, n); b.commit(sid, n)
        live.append(sid)
    for _ in range(60):
        chosen = rng.sample(live, rng.randint(1, len(live)))
        advance = rng.choice([0, 0, 1, 3])
        entries = []
        for sid in chosen:
            q = rng.choice([1, 1, 2, 5, 17])
            if not a.reserve(sid, q + advance):
                continue
            assert b.reserve(sid, q + advance)
            toks = [rng.randrange(1000) for _ in range(q)]
            entries.append((sid, toks, sorted(rng.sample(range(q), rng.randint(0, min(q, 2))))))
        if not entries:
            continue
        need = max(-(-(b.sequences[e[0]].length + advance + len(e[1])) // page) for e in entries)
        pad = rng.choice([0, need, need + 3])
        try:
            want, want_meta, want_order = plain_step(b, entries, pad, advance)
        except plain.CacheError:                       # a new token in a released page (advance beyond the window's edge)
            with pytest.raises(ValueError, match="released"):
                native_step(a, entries, pad, advance)
        else:
            got, meta, order = native_step(a, entries, pad, advance)
            assert order == want_order
            assert np.array_equal(got, want)
            assert (meta[1], meta[4], meta[5], meta[6], meta[7], meta[8], meta[9]) == (
                want_meta["n"], want_meta["max_pages"], want_meta["max_q"], want_meta["max_kv"],
                want_meta["n_single"], want_meta["kv_single"], want_meta["kv_multi"])
        for e in entries:                              # the step "ran": the first tokens are cached
            a.commit(e[0], len(e[1])); b.commit(e[0], len(e[1]))
            rest = a.sequences[e[0]].reserved
            a.commit(e[0], rest); b.commit(e[0], rest)
        a.check_invariants()


def test_step_assembly_refuses_what_does_not_fit():
    m = CacheManager({0: FULL}, page_size=4, num_pages=8, max_seqs=2)
    m.add_sequence("a")
    m.reserve("a", 9)
    with pytest.raises(ValueError, match="too narrow"):
        native_step(m, [("a", [1] * 9, [])], 2, 0)
    with pytest.raises(ValueError, match="too few"):
        native_step(m, [("a", [1] * 13, [])], 0, 0)
    with pytest.raises(ValueError, match="outside"):
        native_step(m, [("a", [1, 2], [2])], 0, 0)
    m.names.key("ghost")
    lib = native.runtime()
    assert lib.iar_step_words(m.handle, 1, native.keys([m.names.find("ghost")]), native.ints([1]), 0, 0, 0) < 0
    assert "not live" in native.last_error()


# ---- scheduler --------------------------------------------------------------------------------
def token_for(request_id, total):
    return (request_id * 31 + total * 7) % 97 + 3


@pytest.mark.parametrize("seed", range(12))
def test_scheduler_takes_the_decisions_of_the_plain_one(seed):
    rng = random.Random(seed)
    page = rng.choice([1, 4, 16])
    num_pages = rng.randint(8, 80) // page + 2
    max_seqs = 6
    options = dict(max_batch_size=rng.randint(1, 6), max_tokens_per_step=rng.choice([4, 16, 64]),
                   prefill_chunk=rng.choice([None, 3, 16]), max_seq_len=rng.choice([24, 48, 4096]),
                   stop_token_ids=[rng.randrange(3, 100), rng.randrange(3, 100)], row_multiple=rng.choice([0, 4, 8, 256]))
    needs = {0: FULL, 1: PagedKV(2, 16, window=rng.choice([6, 20]))} if seed % 2 else {0: FULL}
    ca = CacheManager(needs, page, num_pages, max_seqs)
    cb = plain.CacheManager(needs, page, num_pages, max_seqs)
    sa, sb = Scheduler(ca, **options), plain.Scheduler(cb, **options)
    pending = []
    for i in range(30):
        prompt = [rng.randrange(1, 50) for _ in range(rng.randint(1, min(30, options["max_seq_len"] - 1)))]
        kw = dict(max_tokens=rng.randint(1, 12), bypass_stop_tokens=rng.random() < 0.3,
                  extra_stop_token_ids=(rng.randrange(3, 100),) if rng.random() < 0.3 else ())
        pending.append((Request(i, list(prompt), SamplingParams.greedy(**kw)),
                        plain.Request(i, list(prompt), SimpleNamespace(**kw))))
    every = list(pending)
    steps = 0
    while pending or sb.has_work():
        for _ in range(rng.randint(0, 3)):
            if pending:
                x, y = pending.pop(0)
                sa.add(x); sb.add(y)
        assert sa.has_work() == sb.has_work()
        if sb.has_work():
            pa, pb = sa.plan(), sb.plan()
            assert [(e.request.request_id, e.tokens, e.samples) for e in pa.entries] == \
                   [(e.request.request_id, e.tokens, e.samples) for e in pb.entries]
            assert [r.request_id for r in pa.preempted] == [r.request_id for r in pb.preempted]
            assert [(r.request_id, r.error) for r in pa.failed] == [(r.request_id, r.error) for r in pb.failed]
            assert [r.request_id for r in sa.waiting] == [r.request_id for r in sb.waiting]
            assert [r.request_id for r in sa.running] == [r.request_id for r in sb.running]
            drawn = {e.request.request_id: token_for(e.request.request_id, e.request.total) for e in pb.entries if e.samples}
            da, db = sa.commit(pa, drawn), sb.commit(pb, drawn)
            assert [(r.request_id, r.finish_reason) for r in da] == [(r.request_id, r.finish_reason) for r in db]
            assert [g.pool.num_free for g in ca.groups] == [g.pool.num_free for g in cb.groups]
            ca.check_invariants()
        steps += 1
        assert steps < 20000
    for x, y in every:
        assert (x.status, x.finish_reason, x.error, x.output, x.computed, x.preemptions) == \
               (y.status, y.finish_reason, y.error, y.output, y.computed, y.preemptions)
    assert all(g.pool.num_free == g.pool.num_pages for g in ca.groups) and ca.slots.num_free == max_seqs
    assert len(ca.sequences) == 0 and not ca.names.names()          # no name is left behind


def test_runs_of_decode_steps_commit_like_single_steps():
    cache = CacheManager({0: FULL}, page_size=4, num_pages=32, max_seqs=4)
    s = Scheduler(cache, max_batch_size=4, stop_token_ids=[9])
    a = Request("a", [1, 2, 3], SamplingParams.greedy(max_tokens=6))
    b = Request("b", [4, 5], SamplingParams.greedy(max_tokens=3))
    s.add(a); s.add(b)
    plan = s.plan()
    s.commit(plan, {"a": 11, "b": 12})
    for r in (a, b):
        assert cache.reserve(r.request_id, 3)
    running = s.running
    assert s.commit_decode(running, [21, 22]) == []
    done = s.commit_decode(running, [9, 23])                       # a meets a stop token, b its length
    assert [(r.request_id, r.finish_reason) for r in done] == [("a", "stop"), ("b", "length")]
    assert s.commit_decode(running, [5, 5]) == []                  # both are finished: passed over
    assert a.output == [11, 21, 9] and b.output == [12, 22, 23] and not s.has_work()
    assert cache.groups[0].pool.num_free == 32
