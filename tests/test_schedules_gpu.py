"""Schedules of the decode path that the replay traces do not reach: captured graphs across a context
bucket's boundary, a staging buffer that grows after graphs were captured, more shapes than graphs are
kept, preemption under seeded draws and in bfloat16, and a window whose passed pages hold NaN."""
import io
import os

import numpy as np
import pytest
import torch

import plain_model as pm
import trace_modes as tm
from tiny_configs import TINY, random_tokens, write_model

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    out = {}
    for name in ("A", "B", "D"):
        folder = write_model(str(tmp_path_factory.mktemp(f"sched_{name}")), TINY[name], seed=33)
        out[name] = (folder, *pm.read_model(folder, torch.float64))
    return out


def forced_decode(eng, prompts, tails):
    """Prompts in one step each, then the given tokens one step at a time for all requests together; returns
    the logits of every decode step [steps][requests, vocab] (copies) and the replay count after each."""
    from inferrs_amd.engine import Entry
    for rid, p in prompts.items():
        eng.step([Entry(rid, p, [])])
    rows, replays = [], []
    steps = len(next(iter(tails.values())))
    for i in range(steps):
        rows.append(eng.step([Entry(rid, [tails[rid][i]], [0]) for rid in prompts]).clone())
        replays.append(eng.graph_replays)
    for rid in prompts:
        eng.end_request(rid)
    return rows, replays


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_across_a_bucket_boundary(tiny, dtype):
    """Three requests whose lengths pass 1,024 tokens (the end of a captured graph's context bucket) at different
    steps: every step's logits equal those of an engine without graphs, on both sides of the boundary, and
    graphs were replayed on both sides."""
    from inferrs_amd.engine import Engine
    folder, cfg, params = tiny["D"]
    vocab = TINY["D"]["vocab_size"]
    lengths = {"a": 1000, "b": 1015, "c": 980}
    steps = 60
    seqs = {r: random_tokens(n + steps, vocab, 900 + n) for r, n in lengths.items()}
    prompts = {r: seqs[r][:lengths[r]] for r in seqs}
    tails = {r: seqs[r][lengths[r]:] for r in seqs}
    pages = sum(-(-(n + steps) // 16) for n in lengths.values()) + 2
    outs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=pages, max_seqs=4, use_graphs=graphs)
        assert eng.use_graphs == graphs
        outs[graphs] = forced_decode(eng, prompts, tails)
        eng.cache.check_invariants()
    rows_g, replays = outs[True]
    rows_e, none = outs[False]
    assert none[-1] == 0
    crossing = 1024 - 1015                    # the step whose longest request reaches 1,025 tokens with its new one
    assert replays[crossing - 1] >= crossing - 2 and replays[-1] - replays[crossing + 1] >= steps - crossing - 4
    assert replays[crossing] == replays[crossing - 1]           # the first step of the new bucket runs eagerly
    scale = max(float(r.abs().max()) for r in rows_e)
    worst = max(float((g - e).abs().max()) for g, e in zip(rows_g, rows_e)) / scale
    # 32-bit: the same sums in the same order.  bfloat16: a graph's step sees the bucket's width, an eager step the
    # longest request, so the keys may be split between waves in another way: rounding only
    assert worst <= (1e-6 if dtype == "float32" else 2e-2), worst
    # and both are the plain model's logits
    ref = pm.forward(cfg, params, seqs["b"])
    got = torch.stack([r[1] for r in rows_g]).cpu().double()
    err = float((got - ref[lengths["b"]:lengths["b"] + steps]).abs().max() / ref.abs().max())
    assert err <= (1e-5 if dtype == "float32" else 3e-2), err


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_runs_of_decode_steps_across_a_bucket_boundary(tiny, dtype):
    """The generation loop queues eight decode steps at a time; a run never straddles a bucket, and the tokens
    are those of single steps (32-bit: of an engine without graphs)."""
    from inferrs_amd.engine import Engine, GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["D"]
    vocab = TINY["D"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 950 + n) for n in (1003, 990, 1011)]
    results = {}
    for mode, graphs, run in (("runs", True, 8), ("single", True, 1), ("eager", False, 1)):
        if mode == "eager" and dtype != "float32":
            continue
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=3 * 68 + 2, max_seqs=4, use_graphs=graphs)
        loop = GenerationLoop(eng, decode_run=run, stop_token_ids=[])
        reqs = [loop.add(p, SamplingParams.greedy(max_tokens=60)) for p in prompts]
        loop.run()
        results[mode] = [list(r.output) for r in reqs]
        if mode == "runs":
            assert eng.graph_replays > 40
        eng.cache.check_invariants()
        assert not eng.cache.sequences
    assert all(len(o) == 60 for o in results["runs"])
    if dtype == "float32":
        assert results["runs"] == results["single"] == results["eager"]
        return
    # bfloat16: a run that would end beyond the boundary is not queued, so near the boundary the two ways take the
    # old bucket's graph for different steps, and a graph of a wider bucket may split the keys between waves in
    # another way: rounding.  Where the tokens part, the two choices' logits are as close as that (in 32-bit).
    from inferrs_amd.engine import Entry
    exact = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=70, max_seqs=1, use_graphs=False)
    for prompt, a, b in zip(prompts, results["runs"], results["single"]):
        if a == b:
            continue
        i = next(j for j in range(60) if a[j] != b[j])
        row = exact.step([Entry("x", prompt + a[:i], [len(prompt) + i - 1])])[0]
        exact.end_request("x")
        assert abs(float(row[a[i]] - row[b[i]])) < 0.02, f"token {i}: {a[i]} against {b[i]}, logits {float(row[a[i]])} and {float(row[b[i]])}"
        assert float(row.max() - max(row[a[i]], row[b[i]])) < 0.02


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_staging_buffer_that_grows_drops_the_captured_graphs(tiny, dtype):
    """Graphs hold the address of the step's device buffer.  A later, longer prompt portion makes that buffer
    grow and move: the graphs captured before are dropped, and decode steps afterwards still give the
    logits of an engine without graphs."""
    from inferrs_amd.engine import Engine, Entry
    folder, cfg, params = tiny["D"]
    vocab = TINY["D"]["vocab_size"]
    short, long_prompt = random_tokens(40, vocab, 1), random_tokens(1500, vocab, 2)
    tail = random_tokens(12, vocab, 3)
    outs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=120, max_seqs=4, use_graphs=graphs)
        eng.step([Entry("s", short, [])])
        rows = [eng.step([Entry("s", [t], [0])]).clone() for t in tail[:6]]
        generation, replays = eng.builder.generation, eng.graph_replays
        if graphs:
            assert replays >= 4
        eng.step([Entry("l", long_prompt, [])])                     # 1,500 tokens: more words than the buffer had
        assert eng.builder.generation > generation
        rows += [eng.step([Entry("s", [t], [0])]).clone() for t in tail[6:]]
        if graphs:
            assert eng.graph_replays >= replays + 4                 # captured again over the new buffer, and replayed
        outs[graphs] = rows
    scale = max(float(r.abs().max()) for r in outs[False])
    worst = max(float((g - e).abs().max()) for g, e in zip(outs[True], outs[False])) / scale
    assert worst <= (1e-6 if dtype == "float32" else 2e-2), worst


def test_more_shapes_than_graphs_are_kept(tiny):
    """A batch that shrinks request by request, with room for three graphs only: old ones are dropped, every
    step still equals the eager one."""
    from inferrs_amd.engine import Engine, Entry
    folder, cfg, params = tiny["B"]
    vocab = TINY["B"]["vocab_size"]
    seqs = {f"r{i}": random_tokens(20 + 3 * i + 40, vocab, 40 + i) for i in range(6)}
    outs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=80, max_seqs=6, use_graphs=graphs)
        eng.MAX_GRAPHS = 3
        live = {r: 20 + 3 * i for i, r in enumerate(seqs)}
        for r, n in live.items():
            eng.step([Entry(r, seqs[r][:n], [])])
        rows = []
        for step in range(36):
            if step and step % 6 == 0:                              # a request ends: another shape from here on
                gone = sorted(live)[-1]
                eng.end_request(gone)
                del live[gone]
            rows.append(eng.step([Entry(r, [seqs[r][n]], [0]) for r, n in live.items()]).clone())
            live = {r: n + 1 for r, n in live.items()}
            assert len(eng._graphs) <= 3
        outs[graphs] = rows
        if graphs:
            assert eng.graph_replays >= 6 * 4
    assert all(torch.equal(g, e) for g, e in zip(outs[True], outs[False]))


def test_preemption_under_seeded_draws_gives_the_same_tokens(tiny):
    """A pool so tight that requests are preempted and recomputed: with temperature and fixed seeds the tokens
    are those of a roomy pool (a draw depends on the seed and the token's index, not on when it is made)."""
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["A"]
    vocab = TINY["A"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 190 + n) for n in (20, 24, 28, 18)]
    sp = [SamplingParams(temperature=0.8, top_k=0, top_p=0.95, repetition_penalty=1.1, seed=70 + i, max_tokens=24,
                         bypass_stop_tokens=True) for i in range(4)]
    roomy = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=256, max_seqs=4)
    want = roomy.generate(prompts, sp)
    tight = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=30, max_seqs=4)
    got = tight.generate(prompts, sp)
    assert sum(g.preemptions for g in got) > 0 and sum(g.preemptions for g in want) == 0
    assert [g.tokens for g in got] == [g.tokens for g in want]
    tight.cache.check_invariants()


def test_preemption_in_bfloat16_stays_with_the_plain_model(tiny):
    """bfloat16 under a tight pool: a recomputed request's keys come from a prompt portion's kernels instead of
    decode steps', so its logits move by rounding; greedy tokens agree with the plain model's wherever its two
    best logits are further apart than that."""
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["A"]
    vocab = TINY["A"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 290 + n) for n in (20, 24, 28, 18)]
    tight = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=8, max_seqs=4)     # 128 slots for ~186 tokens
    got = tight.generate(prompts, SamplingParams.greedy(max_tokens=24, bypass_stop_tokens=True))
    assert sum(g.preemptions for g in got) > 0 and all(g.finish_reason == "length" for g in got)
    for prompt, out in zip(prompts, got):
        toks = list(prompt)
        for i, t in enumerate(out.tokens):
            row = pm.forward(cfg, params, toks)[-1]
            top = torch.topk(row, 2)
            if t != int(top.indices[0]):
                assert float(top.values[0] - top.values[1]) < 0.02, f"token {i}: {t} against {int(top.indices[0])}"
                break
            toks.append(t)
    tight.cache.check_invariants()
    assert not tight.cache.sequences


def test_captured_decode_steps_of_more_rows_than_the_own_products_take():
    """160 requests decode together: their products go to the vendor's library, called directly, inside the captured
    graph as in the eager step (every replay against the eager engine, bit for bit)."""
    import torch
    from inferrs_amd.config import Qwen3Config
    from inferrs_amd.engine import Engine, Entry
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=1000, hidden_size=256,
               intermediate_size=512, num_hidden_layers=2, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
               rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=512)
    outs = {}
    for graphs in (False, True):
        eng = Engine.from_random(Qwen3Config.from_dict(raw), seed=1, dtype="bfloat16", page_size=16, num_pages=200,
                                 max_seqs=170, use_graphs=graphs)
        ids = [f"r{i}" for i in range(160)]
        eng.step([Entry(r, [1 + i % 7, 2, 3, 4 + i % 5], [3]) for i, r in enumerate(ids)])
        rows = [eng.step([Entry(r, [10 + step], [0]) for r in ids]).clone() for step in range(5)]
        outs[graphs] = torch.stack(rows)
        assert (eng.graph_replays >= 3) == graphs
    assert torch.equal(outs[True], outs[False])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_portions_of_a_prompt_across_a_bucket_boundary(tiny, dtype):
    """Steps of few tokens are captured like decode steps where the host is their bound (forced here: the share of the
    host that a capture asks for is set to nothing).  A prompt of 1,250 tokens in portions of 50 beside nothing else:
    the shape repeats, so its first two steps run eagerly and the steps from the third on are replayed, until the
    portion that passes 1,024 tokens starts another bucket.  The logits at every portion's first and last token are
    those of an engine without graphs and of the plain model."""
    from inferrs_amd.engine import Engine, Entry
    folder, cfg, params = tiny["D"]
    vocab = TINY["D"]["vocab_size"]
    total, portion = 1250, 50
    toks = random_tokens(total, vocab, 77)
    outs, replays = {}, []
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=total // 16 + 3, max_seqs=2, use_graphs=graphs)
        eng.GRAPH_HOST_SHARE = 0.0
        rows = []
        for lo in range(0, total, portion):
            rows.append(eng.step([Entry("p", toks[lo:lo + portion], [0, portion - 1])]).clone())
            if graphs:
                replays.append(eng.graph_replays)
        eng.end_request("p")
        eng.cache.check_invariants()
        assert graphs or eng.graph_replays == 0
        outs[graphs] = torch.cat(rows)
    crossing = 1024 // portion                  # the portion that holds token 1,024
    assert replays[1] == 0 and replays[crossing - 1] == crossing - 2           # eager, eager and timed, captured and replayed, replayed ...
    assert replays[crossing + 1] == replays[crossing - 1]                      # another bucket: eager again
    assert replays[-1] == replays[crossing - 1] + total // portion - crossing - 2
    scale = float(outs[False].abs().max())
    worst = float((outs[True] - outs[False]).abs().max()) / scale
    assert worst <= (1e-6 if dtype == "float32" else 2e-2), worst
    ref = pm.forward(cfg, params, toks)
    at = [p for lo in range(0, total, portion) for p in (lo, lo + portion - 1)]
    err = float((outs[True].cpu().double() - ref[at]).abs().max() / ref.abs().max())
    assert err <= (1e-5 if dtype == "float32" else 3e-2), err


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_mixed_steps_equal_eager_ones(tiny, dtype):
    """Two requests decode while others bring their prompts in portions of 24 tokens beside them: the mixed step's
    shape repeats and is replayed from a graph from its third step on; between the rounds requests end and their pages go to the next.
    Every step's logits are those of an engine without graphs, and the decoding requests' those of the plain model."""
    from inferrs_amd.engine import Engine, Entry
    folder, cfg, params = tiny["B"]
    vocab = TINY["B"]["vocab_size"]
    rounds, portion, portions = 4, 24, 3
    deco = {r: random_tokens(30 + rounds * portions + 2, vocab, 500 + i) for i, r in enumerate(("a", "b"))}
    prompts = [random_tokens(portion * portions, vocab, 600 + i) for i in range(rounds)]
    outs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=8, num_pages=40, max_seqs=4, use_graphs=graphs)
        eng.GRAPH_HOST_SHARE = 0.0                       # (captured whatever the host's share of the step)
        eng.step([Entry(r, t[:30], []) for r, t in deco.items()])
        at, rows = 30, []
        for k, prompt in enumerate(prompts):
            for j in range(portions):
                entries = [Entry(f"p{k}", prompt[j * portion:(j + 1) * portion], [portion - 1])]
                entries[1:1] = [Entry(r, [t[at]], [0]) for r, t in deco.items()]      # (the portion first, as a caller may give it)
                rows.append(eng.step(entries).clone())
                at += 1
            eng.end_request(f"p{k}")
        eng.cache.check_invariants()
        if graphs:
            assert eng.graph_replays >= rounds * portions - 2
        outs[graphs] = rows
    scale = max(float(r.abs().max()) for r in outs[False])
    worst = max(float((g - e).abs().max()) for g, e in zip(outs[True], outs[False])) / scale
    assert worst <= (1e-6 if dtype == "float32" else 2e-2), worst
    for i, (r, t) in enumerate(deco.items()):
        ref = pm.forward(cfg, params, t)
        got = torch.stack([row[1 + i] for row in outs[True]]).cpu().double()
        err = float((got - ref[30:30 + rounds * portions]).abs().max() / ref.abs().max())
        assert err <= (1e-5 if dtype == "float32" else 3e-2), err
    ref = pm.forward(cfg, params, prompts[-1])
    got = torch.stack([row[0] for row in outs[True][-portions:]]).cpu().double()
    err = float((got - ref[[portion - 1, 2 * portion - 1, 3 * portion - 1]]).abs().max() / ref.abs().max())
    assert err <= (1e-5 if dtype == "float32" else 3e-2), err


def test_a_shape_whose_step_the_gpu_bounds_stays_eager(tiny):
    """The capture of a step other than a decode step is decided by a measurement: with a share that no host can
    reach the shape is marked eager at its third step and never captured, and its logits are the same."""
    from inferrs_amd.engine import Engine, Entry
    folder, cfg, params = tiny["A"]
    vocab = TINY["A"]["vocab_size"]
    prompt = random_tokens(40, vocab, 9)
    eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=8, max_seqs=2)
    eng.GRAPH_HOST_SHARE = 1e9
    rows = []
    for _ in range(5):
        rows.append(eng.step([Entry("p", prompt, [39])]).clone())
        eng.end_request("p")
    assert eng.graph_replays == 0 and not eng._graphs and list(eng._seen.values()) == ["eager"]
    assert all(torch.equal(rows[0], r) for r in rows[1:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_portions_that_want_no_logits(tiny, dtype):
    """Portions in the middle of a prompt ask for no logits: their shape (no wanted row) is captured and replayed like
    any other, the cache they leave is the same, and the last portion's logits are those of an engine without graphs."""
    from inferrs_amd.engine import Engine, Entry
    folder, cfg, params = tiny["A"]
    vocab = TINY["A"]["vocab_size"]
    toks = random_tokens(220, vocab, 5)
    outs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=16, max_seqs=2, use_graphs=graphs)
        eng.GRAPH_HOST_SHARE = 0.0
        for lo in range(0, 200, 20):
            empty = eng.step([Entry("p", toks[lo:lo + 20], [])])
            assert tuple(empty.shape) == (0, vocab)
        outs[graphs] = eng.step([Entry("p", toks[200:], [0, 19])]).clone()
        assert eng.graph_replays == (8 if graphs else 0)
    scale = float(outs[False].abs().max())
    assert float((outs[True] - outs[False]).abs().max()) / scale <= (1e-6 if dtype == "float32" else 2e-2)
    ref = pm.forward(cfg, params, toks)
    err = float((outs[True].cpu().double() - ref[[200, 219]]).abs().max() / ref.abs().max())
    assert err <= (1e-5 if dtype == "float32" else 3e-2), err


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_that_shrinks_request_by_request_meets_few_shapes(tiny, dtype):
    """13 requests decode and one after the other ends: the steps of 13, 12, 11, 10 and 9 requests run on the graphs
    of 14, 12 and 10 rows (the missing rows are a hidden request's, which lives inside a step only).  Every step's
    logits are those of an engine without graphs, whose steps have no such rows; nothing of the hidden request is left."""
    from inferrs_amd.engine import Engine, Entry
    from inferrs_amd.engine.engine import _PAD
    folder, cfg, params = tiny["B"]
    vocab = TINY["B"]["vocab_size"]
    assert [Engine.padded_batch(n) for n in (1, 8, 9, 10, 13, 16, 17, 33, 100, 129)] == [1, 8, 10, 10, 14, 16, 20, 40, 112, 160]
    seqs = {f"r{i:02d}": random_tokens(12 + 2 * i + 30, vocab, 70 + i) for i in range(13)}
    outs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=8, num_pages=13 * 9 + 2, max_seqs=13, use_graphs=graphs)
        live = {r: 12 + 2 * i for i, r in enumerate(seqs)}
        for r, n in live.items():
            eng.step([Entry(r, seqs[r][:n], [])])
        rows = []
        for step in range(25):
            if step and step % 5 == 0:
                gone = sorted(live)[-1]
                eng.end_request(gone)
                del live[gone]
            got = eng.step([Entry(r, [seqs[r][n]], [0]) for r, n in live.items()])
            assert got.shape[0] == len(live)
            rows.append(got.clone())
            live = {r: n + 1 for r, n in live.items()}
            assert not eng.has_request(_PAD)
        eng.cache.check_invariants()
        if graphs:
            assert sorted(k[0] for k in eng._graphs if k[4] == 1) == [10, 12, 14] and eng.graph_replays >= 25 - 3
        for r in live:
            eng.end_request(r)
        assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups) and not eng.cache.sequences
        outs[graphs] = rows
    scale = max(float(r.abs().max()) for r in outs[False])
    worst = max(float((g - e).abs().max()) for g, e in zip(outs[True], outs[False])) / scale
    assert worst <= (1e-6 if dtype == "float32" else 2e-2), worst
    ref = pm.forward(cfg, params, seqs["r00"])
    got = torch.stack([r[0] for r in outs[True]]).cpu().double()
    err = float((got - ref[12:12 + 25]).abs().max() / ref.abs().max())
    assert err <= (1e-5 if dtype == "float32" else 3e-2), err


def test_a_pool_without_a_page_to_spare_runs_the_batch_as_it_is(tiny):
    """The hidden request's rows need a page; where the callers' requests hold them all, the step runs with the rows
    it has."""
    from inferrs_amd.engine import Engine, Entry
    folder, cfg, params = tiny["B"]
    vocab = TINY["B"]["vocab_size"]
    seqs = [random_tokens(7 + 6, vocab, 90 + i) for i in range(9)]
    eng = Engine.from_folder(folder, dtype="bfloat16", page_size=8, num_pages=9 * 2, max_seqs=9)
    for i, t in enumerate(seqs):
        eng.step([Entry(i, t[:7], [])])
    rows = []
    for s in range(6):                                   # (from the second token on every request holds its two pages)
        rows.append(eng.step([Entry(i, [t[7 + s]], [0]) for i, t in enumerate(seqs)]).clone())
    assert [k[0] for k in eng._graphs if k[4] == 1] == [9] and eng.graph_replays >= 3      # (k[4]: the longest portion; 1 for decode steps)
    ref = pm.forward(cfg, params, seqs[4])
    got = torch.stack([r[4] for r in rows]).cpu().double()
    assert float((got - ref[7:13]).abs().max() / ref.abs().max()) <= 3e-2


def test_runs_of_decode_steps_with_rows_of_the_hidden_request(tiny):
    """The generation loop queues runs of decode steps of 11 requests (graphs of 12 rows) that draw with seeds: the
    tokens are those of single steps and of an engine without graphs' arithmetic, the hidden request's row is never seen."""
    from inferrs_amd.engine import Engine, GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["A"]
    vocab = TINY["A"]["vocab_size"]
    prompts = [random_tokens(6 + i, vocab, 30 + i) for i in range(11)]
    results = {}
    for run in (1, 4):
        eng = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=11 * 3 + 2, max_seqs=11)
        loop = GenerationLoop(eng, decode_run=run, max_batch_size=11, stop_token_ids=[])
        reqs = [loop.add(p, SamplingParams(temperature=0.9, top_k=20, seed=5 + i, max_tokens=18)) for i, p in enumerate(prompts)]
        loop.run()
        results[run] = [list(r.output) for r in reqs]
        assert eng.graph_replays >= 10 and all(k[0] == 12 for k in eng._graphs if k[4] == 1 and k[0] > 8)
        eng.cache.check_invariants()
        assert not eng.cache.sequences
    assert results[4] == results[1] and all(len(o) == 18 for o in results[1])


def test_a_run_of_decode_steps_that_loses_its_hidden_rows_falls_back_to_single_steps(tiny):
    """Nine requests decode on the graph of ten rows.  When the pages that a run of eight steps reserves for them are the
    pool's last, the hidden request finds none, the run is not started (`decode_chain` says so) and the loop goes on
    step by step: the tokens are those of a loop that never queues runs."""
    from inferrs_amd.engine import Engine, Entry, GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["A"]
    vocab = TINY["A"]["vocab_size"]
    prompts = [random_tokens(13, vocab, 200 + i) for i in range(9)]
    # the engine alone: the graph of ten rows is there, the pages go to the requests, the run is refused
    eng = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=18, max_seqs=9)
    for i, p in enumerate(prompts):
        eng.step([Entry(i, p, [])])
    for s in range(3):                                   # positions 13, 14, 15: a page each, nine to spare
        eng.step([Entry(i, [1 + s], [0]) for i in range(9)])
    assert [k[0] for k in eng._graphs if k[4] == 1] == [10]
    ids = list(range(9))
    assert eng.chain_ready(ids, 8)
    for i in ids:
        assert eng.cache.reserve(i, 8)
    assert all(g.pool.num_free == 0 for g in eng.cache.groups)
    assert eng.decode_chain(ids, [5] * 9, 8) is None
    eng.cache.check_invariants()
    # the loop: the same tokens with and without runs
    results = {}
    for run in (1, 8):
        eng = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=18, max_seqs=9)
        loop = GenerationLoop(eng, decode_run=run, max_batch_size=9, stop_token_ids=[])
        reqs = [loop.add(p, SamplingParams.greedy(max_tokens=16)) for p in prompts]
        loop.run()
        results[run] = [list(r.output) for r in reqs]
        eng.cache.check_invariants()
        assert not eng.cache.sequences
    assert results[8] == results[1] and all(len(o) == 16 for o in results[1])
