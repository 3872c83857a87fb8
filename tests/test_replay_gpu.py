"""The engine against the plain implementation under every way of cutting the work: each
request alone and whole; most of it in one step and the last 32 tokens one by one; portions of
changing size down to two tokens; and up to four live requests mixed, portions of some beside
decoded tokens of others, in a pool so small that pages are used again.  32-bit and bfloat16.

The plain implementation runs in 64-bit and stands for the exact result.

Tolerances.  32-bit: 1e-5 of the largest logit.  The plain implementation run in 32-bit is
itself 4e-7 to 7e-6 away from the 64-bit result on these models, the engine 3e-7 to 9e-6.  Between two cuttings the 32-bit engine has the same order of sums for every
position (per-row norms, keys walked in tiles aligned to absolute position, a fixed k order in
the products), so they agree to 1e-6 of the scale.  bfloat16: every stored activation is rounded to 8 bits of mantissa, and how far that moves
a logit depends on the model (sharper attention amplifies it).  The bound is therefore measured
on the model itself: the plain implementation run in bfloat16 tensor arithmetic (every
operation rounded, as the reference's CPU path does) against the same in 32-bit, largest
difference over all positions.  The engine keeps more in 32-bit registers than that, so it has to
be at least as close to the 32-bit result (measured: 0.4 to 0.7 of the bound).  Sharpened models
(see `write_model`) make a lost or misplaced key change logits by 10 % and more.  The sharpening
is 2.0 for 32-bit (scores spread 16 times wider) and 1.5 for bfloat16 (5 times): sharper
than that, rounding of queries and keys alone moves the scores so far that the comparison
says little (at 2.5 the plain implementation in 32-bit is 1.5e-5 away from 64-bit)."""
import io
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_model as pm
import trace_modes as tm
from call_counter import CallCounter
from tiny_configs import PAGE_SIZE, TINY, random_tokens, write_model

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = [1, 2, 3, 37, 64, 65, 130, 257, 300]
TOL_PLAIN_F32 = 1e-5
TOL_CROSS_F32 = 1e-6
SHARP = {"float32": 2.0, "bfloat16": 1.5}
# (configuration, sharpened or not)
CASES = [("A", False), ("B", False), ("C", False), ("D", False), ("E", False), ("F", False), ("G", False), ("A", True),
         ("B", True), ("D", True), ("G", True)]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(name, sharpen factor) -> folder, raw config, requests, plain logits."""
    out = {}
    for name, sharp in CASES:
        for sharpen in (sorted(set(SHARP.values())) if sharp else [1.0]):
            raw = TINY[name]
            folder = write_model(str(tmp_path_factory.mktemp(f"model_{name}")), raw, seed=5, sharpen=sharpen)
            cfg, params = pm.read_model(folder, torch.float64)
            reqs = {f"r{i}": random_tokens(n, raw["vocab_size"], 100 + i) for i, n in enumerate(LENGTHS)}
            ref = {r: pm.forward(cfg, params, t).numpy().astype(np.float32) for r, t in reqs.items()}
            out[(name, sharpen)] = (folder, raw, reqs, ref)
    return out


_BF16_BOUND = {}


def bound(folder, reqs, ref, dtype, cross=False):
    """Largest allowed difference as a fraction of the largest logit."""
    if dtype == "float32":
        return TOL_CROSS_F32 if cross else TOL_PLAIN_F32
    if folder not in _BF16_BOUND:
        cfg, params = pm.read_model(folder, torch.bfloat16)
        rounded = {r: pm.forward(cfg, params, t).float().numpy() for r, t in reqs.items()}
        _BF16_BOUND[folder] = worst(rounded, ref, reqs)[0]
    return _BF16_BOUND[folder]


def pick(models, name, sharp, dtype):
    return models[(name, SHARP[dtype] if sharp else 1.0)]


def replay(folder, raw, name, dtype, trace, out_dir, page_size=None):
    from inferrs_amd.engine import Engine, run_trace
    page = page_size or PAGE_SIZE[name]
    eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page),
                             max_seqs=4)
    run_trace(eng, trace.lines, out_dir, io.StringIO())
    eng.cache.check_invariants()
    assert not eng.cache.sequences and all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    return trace.read(out_dir, raw["vocab_size"])


def worst(got, ref, reqs, scale=None):
    if scale is None:
        scale = max(float(np.abs(v).max()) for v in ref.values())
    err, where = 0.0, None
    for r, toks in reqs.items():
        for p in range(len(toks)):
            e = float(np.abs(got[r][p] - ref[r][p]).max())
            if not e <= err:            # also catches NaN
                err, where = e, (r, p)
    return err / scale, where


def traces(reqs):
    return {
        "whole": tm.whole(reqs),
        "tail32": tm.prefix_then_single(reqs, 32),
        "portions": tm.portions(reqs, [7, 2, 16, 3, 2, 33, 5, 2, 64]),
        "mixed": tm.mixed(reqs, seed=1),
        "mixed2": tm.mixed(dict(reversed(list(reqs.items()))), seed=2, max_live=3),
    }


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: c[0] + ("sharp" if c[1] else ""))
def test_every_cutting_matches_plain(models, tmp_path, case, dtype):
    folder, raw, reqs, ref = pick(models, case[0], case[1], dtype)
    first = None
    for mode, trace in traces(reqs).items():
        if mode.startswith("mixed"):
            assert trace.max_live >= 3 and trace.max_tokens < sum(tm.round_up(len(t), 64) for t in reqs.values())
        got = replay(folder, raw, case[0], dtype, trace, str(tmp_path / mode))
        err, where = worst(got, ref, reqs)
        assert err <= bound(folder, reqs, ref, dtype), f"{mode}: {err:.3e} of the scale at {where} against the plain implementation"
        if first is None:
            first = got
        else:
            err, where = worst(got, first, reqs, scale=max(float(np.abs(v).max()) for v in ref.values()))
            assert err <= bound(folder, reqs, ref, dtype, cross=True), f"{mode}: {err:.3e} of the scale at {where} against the whole-request run"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(models, tmp_path, dtype):
    """Three tokens in one step, then three hundred one by one."""
    folder, raw, reqs, ref = pick(models, "B", True, dtype)
    one = {"r8": reqs["r8"]}
    got = replay(folder, raw, "B", dtype, tm.prefix_then_single(one, len(one["r8"]) - 3), str(tmp_path))
    err, where = worst(got, ref, one)
    assert err <= bound(folder, reqs, ref, dtype), f"{err:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_page_sizes(models, tmp_path, dtype):
    """Results do not depend on the page size (1, 3: no power of two, 64: one page a request)."""
    folder, raw, reqs, ref = pick(models, "A", True, dtype)
    for page in (1, 3, 64):
        got = replay(folder, raw, "A", dtype, tm.mixed(reqs, seed=page), str(tmp_path / str(page)), page_size=page)
        err, where = worst(got, ref, reqs)
        assert err <= bound(folder, reqs, ref, dtype), f"page size {page}: {err:.3e} at {where}"


def test_poisoned_free_pages_change_nothing(models, tmp_path):
    """Pages that are free or beyond a request's length are never read: NaN in them is harmless."""
    import torch
    from inferrs_amd.engine import Engine, run_trace
    folder, raw, reqs, ref = pick(models, "B", True, "float32")
    trace = tm.mixed(reqs, seed=3)
    eng = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=-(-trace.max_tokens // 8), max_seqs=4)
    for arr in eng.storage.arrays:
        arr.fill_(float("nan"))
    run_trace(eng, trace.lines, str(tmp_path), io.StringIO())
    err, where = worst(trace.read(str(tmp_path), raw["vocab_size"]), ref, reqs)
    assert err <= TOL_PLAIN_F32, f"{err:.3e} at {where}"
    del torch


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, tmp_path, dtype):
    """bin/trace_run as a user starts it: a child process, steps on standard input, `done`
    lines on standard output, files in --out."""
    folder, raw, reqs, ref = pick(models, "B", True, dtype)
    trace = tm.mixed(reqs, seed=7)
    out_dir = str(tmp_path / "out")
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", out_dir, "--max-tokens", str(trace.max_tokens)],
        input=trace.text(), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {i}" for i in range(len(trace.lines))]
    err, where = worst(trace.read(out_dir, raw["vocab_size"]), ref, reqs)
    assert err <= bound(folder, reqs, ref, dtype), f"{err:.3e} at {where}"


def test_trace_run_reads_a_config_as_the_reference_does(models, tmp_path):
    """The reference reads `attention_bias`, `use_sliding_window`, `hidden_act` and `rope_scaling` without acting on
    them (inferrs-models/src/config.rs:291-292, 468-502).  The engine's entry points refuse such values; the replay
    program, whose logits are compared with the reference's formulas, ignores them too, says so, and writes the logits
    of the same folder without those keys."""
    import json
    import shutil
    folder, raw, reqs, ref = pick(models, "A", False, "float32")
    odd = str(tmp_path / "odd")
    shutil.copytree(folder, odd)
    with open(os.path.join(odd, "config.json")) as f:
        config = json.load(f)
    config.update(attention_bias=True, use_sliding_window=True, sliding_window=8, hidden_act="gelu",
                  rope_scaling={"rope_type": "linear", "factor": 2.0})
    with open(os.path.join(odd, "config.json"), "w") as f:
        json.dump(config, f)
    from inferrs_amd.config import ConfigError
    from inferrs_amd.engine import Engine
    with pytest.raises(ConfigError, match="use_sliding_window"):
        Engine.from_folder(odd, dtype="float32", page_size=4, num_pages=8, max_seqs=1)
    some = {k: reqs[k] for k in ("r3", "r4")}
    trace = tm.whole(some)
    out_dir = str(tmp_path / "out")
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", odd, "--dtype", "float32",
         "--out", out_dir, "--max-tokens", str(trace.max_tokens)],
        input=trace.text(), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "ignored here as well" in proc.stderr and "hidden_act = 'gelu'" in proc.stderr
    err, where = worst(trace.read(out_dir, raw["vocab_size"]), ref, some)
    assert err <= TOL_PLAIN_F32, f"{err:.3e} at {where}"


def test_out_of_pages_is_an_error_and_takes_nothing(models):
    from inferrs_amd.cache import OutOfPages
    from inferrs_amd.engine import Engine, Entry
    folder, raw, reqs, _ = pick(models, "A", False, "float32")
    eng = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=4, max_seqs=2)
    with pytest.raises(OutOfPages):
        eng.step([Entry("x", reqs["r3"], [0])])          # 37 tokens into 16 slots
    eng.cache.check_invariants()
    assert not eng.has_request("x") and eng.cache.groups[0].pool.num_free == 4
    eng.step([Entry("y", reqs["r3"][:16], [15])])
    with pytest.raises(OutOfPages):
        eng.step([Entry("y", [1], [0])])
    assert eng.cached_length("y") == 16


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_equal_eager_ones(models, tmp_path, dtype):
    """Decode steps are replayed from a captured graph from the third step of a shape on.  Every
    replay is checked against the same trace run without graphs, with eager steps (portions of
    prompts, other batch sizes) in between the replays."""
    from inferrs_amd.engine import Engine, run_trace
    folder, raw, reqs, ref = pick(models, "D", True, dtype)
    some = {k: reqs[k] for k in ("r3", "r5", "r6", "r7")}
    trace = tm.mixed(some, seed=11, max_live=3, decode_tail=40)
    outs = {}
    for graphs in (False, True):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-trace.max_tokens // 16), max_seqs=4,
                                 use_graphs=graphs)
        run_trace(eng, trace.lines, str(tmp_path / str(graphs)), io.StringIO())
        outs[graphs] = trace.read(str(tmp_path / str(graphs)), raw["vocab_size"])
        assert (eng.graph_replays > 20) == graphs
    scale = max(float(np.abs(v).max()) for v in ref.values())
    err, where = worst(outs[True], outs[False], some, scale=scale)
    # the same kernels with the same arguments, except that the keys may be split differently
    assert err <= (1e-6 if dtype == "float32" else bound(folder, reqs, ref, dtype)), f"{err:.3e} at {where}"
    err, where = worst(outs[True], ref, some, scale=scale)
    assert err <= bound(folder, reqs, ref, dtype), f"{err:.3e} at {where}"


@pytest.mark.parametrize("name,drop", [("B", True), ("A", False)])
def test_logits_head_follows_the_tensor_present(tmp_path, name, drop):
    """`lm_head.weight` is used when the file has it and the embedding table when it has not,
    whatever `tie_word_embeddings` says (inferrs-models/src/models/qwen3.rs:369-372)."""
    from safetensors.torch import load_file, save_file
    from inferrs_amd.engine import Engine, Entry
    folder = write_model(str(tmp_path / "m"), TINY[name], seed=8)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    if drop:
        assert not TINY[name]["tie_word_embeddings"]
        del tensors["lm_head.weight"]                    # untied by its config, but the head is absent
    else:
        assert TINY[name]["tie_word_embeddings"]
        tensors["lm_head.weight"] = torch.randn_like(tensors["model.embed_tokens.weight"].float()).mul(0.02).bfloat16()
    save_file(tensors, path)
    cfg, params = pm.read_model(folder, torch.float64)
    toks = random_tokens(21, TINY[name]["vocab_size"], 4)
    want = pm.forward(cfg, params, toks).numpy()
    eng = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=4, max_seqs=1)
    got = eng.step([Entry("a", toks, list(range(21)))]).cpu().numpy()
    assert float(np.abs(got - want).max()) <= 1e-5 * float(np.abs(want).max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_in_every_cutting(tmp_path, dtype):
    """A 2,500-token request with the serving head size: whole; in portions of 512 beside a
    second request; and its last 40 tokens decoded one by one (through the split-key kernel and,
    from the third step on, a captured graph).  Sharpened attention makes every query depend on a
    few keys that may lie thousands of positions back."""
    from inferrs_amd.engine import Engine, run_trace
    raw = dict(TINY["D"], max_position_embeddings=4096)
    folder = write_model(str(tmp_path / "m"), raw, seed=9, sharpen=SHARP[dtype])
    cfg, params = pm.read_model(folder, torch.float64)
    long_req = random_tokens(2500, raw["vocab_size"], 77)
    other = random_tokens(300, raw["vocab_size"], 78)
    ref = pm.forward(cfg, params, long_req).numpy().astype(np.float32)
    watch = list(range(0, 2500, 97)) + list(range(2440, 2500))
    scale = float(np.abs(ref).max())
    if dtype == "float32":
        limit = TOL_PLAIN_F32
    else:
        cfg_b, params_b = pm.read_model(folder, torch.bfloat16)
        rounded = pm.forward(cfg_b, params_b, long_req).float().numpy()
        limit = float(np.abs(rounded[watch] - ref[watch]).max()) / scale

    def run(trace, name):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-trace.max_tokens // 16), max_seqs=2)
        run_trace(eng, trace.lines, str(tmp_path / name), io.StringIO())
        return trace.read(str(tmp_path / name), raw["vocab_size"])["long"]

    whole = tm.Trace()
    whole.step([("long", long_req, watch)], end=["long"])
    cut = tm.Trace()
    for i in range(0, 2460, 512):
        part = long_req[i:min(i + 512, 2460)]
        entries = [("long", part, [w - i for w in watch if i <= w < i + len(part)])]
        if i == 512:
            entries.append(("other", other, []))
        cut.step(entries, end=["other"] if i == 1024 else [])
    for i in range(2460, 2500):
        cut.step([("long", long_req[i:i + 1], [0])], end=["long"] if i == 2499 else [])
    for name, trace in (("whole", whole), ("cut", cut)):
        got = run(trace, name)
        err = max(float(np.abs(got[w] - ref[w]).max()) for w in watch) / scale
        assert err <= limit, f"{name}: {err:.3e} of the scale, the bound is {limit:.3e}"


@pytest.mark.parametrize("n_req", [14, 24])
def test_captured_steps_of_many_requests_equal_eager_ones(models, tmp_path, n_req):
    """More than 16 requests decode through the vendor's GEMM, and those calls are captured into
    the graph too; 13 to 16 decode through the skinny products, which then sum and norm the stream.
    Every replay must equal the eager step, with eager steps and synchronisations in between."""
    from inferrs_amd.engine import Engine, Entry
    folder, raw, reqs, ref = pick(models, "D", False, "bfloat16")
    n_steps = 14
    prompts = [random_tokens(5 + 3 * i, raw["vocab_size"], 500 + i) for i in range(n_req)]
    feeds = [random_tokens(n_steps, raw["vocab_size"], 600 + i) for i in range(n_req)]
    outs = {}
    for graphs in (False, True):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=n_req * 8 + 4, max_seqs=n_req + 1,
                                 use_graphs=graphs)
        for i, p in enumerate(prompts):
            eng.step([Entry(i, p, [])])
        rows = []
        for s in range(n_steps):
            logits = eng.step([Entry(i, [feeds[i][s]], [0]) for i in range(n_req)])
            rows.append(logits.cpu().numpy().copy())
            if s % 4 == 1:                       # an eager step of another shape between the replays
                eng.step([Entry("extra", random_tokens(9, raw["vocab_size"], s), [8])])
                eng.end_request("extra")
        outs[graphs] = rows
        assert (eng.graph_replays >= n_steps - 2) == graphs
    # the captured step pads its block tables to the bucket, which may split the keys differently:
    # the two runs agree to bfloat16 rounding, and every replay alike (a replay gone wrong is far off)
    scale = max(float(np.abs(o).max()) for o in outs[False])
    errs = [float(np.abs(outs[True][s] - outs[False][s]).max()) / scale for s in range(n_steps)]
    assert max(errs) <= 2 ** -6, f"replays differ from eager steps: {errs}"


@pytest.mark.parametrize("hidden,heads,intermediate", [(4096, 32, 12288), (5120, 40, 17408)], ids=["8B", "14B"])
def test_real_layer_sizes(tmp_path, hidden, heads, intermediate):
    """One layer with the sizes of Qwen3-8B (hidden 4096, 32 query and 8 key/value heads of 128,
    intermediate 12288) or Qwen3-14B (5120, 40 query heads: five a key/value head, 17408) and a small
    vocabulary: the kernels' serving shapes (the skinny products of 6144, 4096 and 2 x 12288 rows, among
    them the variant that stages the activations; at the 14B sizes blocks of 10 and 14 features, k shared
    out between five and seven waves, rows of 512 sums of squares; attention over head size 128) against
    the plain implementation, whole, with a decoded tail and mixed.  bfloat16 within 2 % of the largest
    logit (the tiny models' measured bounds are 1 to 3 %), 32-bit within 1e-5."""
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=1031, hidden_size=hidden,
               intermediate_size=intermediate, num_hidden_layers=1, num_attention_heads=heads, num_key_value_heads=8,
               head_dim=128, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
               max_position_embeddings=4096, hidden_act="silu")
    folder = write_model(str(tmp_path / "layer"), raw, seed=21)
    cfg, params = pm.read_model(folder, torch.float64)
    reqs = {f"r{i}": random_tokens(n, raw["vocab_size"], 300 + i) for i, n in enumerate([3, 40, 90])}
    ref = {r: pm.forward(cfg, params, t).numpy().astype(np.float32) for r, t in reqs.items()}
    del params
    from inferrs_amd.engine import Engine, run_trace
    for dtype, tol in (("bfloat16", 2e-2), ("float32", TOL_PLAIN_F32)):
        for mode, trace in (("whole", tm.whole(reqs)), ("tail", tm.prefix_then_single(reqs, 6)),
                            ("mixed", tm.mixed(reqs, seed=3, max_live=3, decode_tail=5))):
            eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-trace.max_tokens // 16) + 1, max_seqs=4)
            out_dir = str(tmp_path / f"{dtype}_{mode}")
            run_trace(eng, trace.lines, out_dir, io.StringIO())
            eng.cache.check_invariants()
            got = trace.read(out_dir, raw["vocab_size"])
            err, where = worst(got, ref, reqs)
            assert err <= tol, f"{dtype} {mode}: {err:.3e} at {where}"
            del eng
            torch.cuda.empty_cache()


def test_own_large_products_through_the_engine(models, tmp_path):
    """The model without the vendor's GEMM: every cutting with the package's own tiled kernel for the products of
    many rows (widths that are multiples of 64: tiny configuration A; other widths stay with the library)."""
    from inferrs_amd import ops
    folder, raw, reqs, ref = pick(models, "A", False, "bfloat16")
    limit = bound(folder, reqs, ref, "bfloat16")
    calls = []
    saved, ops.LARGE_PRODUCTS, inner = ops.LARGE_PRODUCTS, "own", ops.gemm_mfma_bf16
    ops.gemm_mfma_bf16 = lambda *a, **k: (calls.append(1), inner(*a, **k))[1]
    try:
        for mode, trace in traces(reqs).items():
            got = replay(folder, raw, "A", "bfloat16", trace, str(tmp_path / f"own_{mode}"))
            err, where = worst(got, ref, reqs)
            assert err <= limit, f"{mode}: {err:.3e} at {where}"
    finally:
        ops.LARGE_PRODUCTS, ops.gemm_mfma_bf16 = saved, inner
    assert calls, "the tiled kernel never ran"


def test_real_layer_sizes_long_prompt_in_portions(tmp_path):
    """The same layer over a prompt of 1,100 tokens, whole and in portions of 300, 37 and 512 tokens: with head
    size 128 these steps take the attention kernel of four-wave blocks, and the late portions (few tiles, more
    than 1,024 keys) its form that shares the keys out between blocks and merges them."""
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=1031, hidden_size=4096,
               intermediate_size=12288, num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8,
               head_dim=128, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
               max_position_embeddings=4096, hidden_act="silu")
    folder = write_model(str(tmp_path / "layer8b"), raw, seed=22)
    cfg, params = pm.read_model(folder, torch.float64)
    reqs = {"long": random_tokens(1100, raw["vocab_size"], 400)}
    ref = {r: pm.forward(cfg, params, t).numpy().astype(np.float32) for r, t in reqs.items()}
    del params
    from inferrs_amd.engine import Engine, run_trace
    for mode, trace in (("whole", tm.whole(reqs)), ("portions", tm.portions(reqs, (300, 37, 512)))):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=-(-trace.max_tokens // 16) + 1, max_seqs=2)
        out_dir = str(tmp_path / mode)
        run_trace(eng, trace.lines, out_dir, io.StringIO())
        eng.cache.check_invariants()
        got = trace.read(out_dir, raw["vocab_size"])
        err, where = worst(got, ref, reqs)
        assert err <= 2e-2, f"{mode}: {err:.3e} at {where}"
        del eng
        torch.cuda.empty_cache()


@pytest.fixture(scope="module")
def many_requests(models):
    """100 requests of different lengths on configuration G (widths in steps of 128, head size 128: the products of 17 to
    128 rows run on the kernels made for them, the two of 1,024 inputs split along k), each a prompt and 12 tokens that
    are fed one by one whatever the model would choose; the plain implementation's logits at the fed places, and the
    bfloat16 bound measured on these very sequences."""
    folder, raw, _, _ = models[("G", 1.0)]
    n_steps = 12
    prompts = [random_tokens(3 + (7 * i) % 61 + i % 64, raw["vocab_size"], 900 + i) for i in range(100)]
    feeds = [random_tokens(n_steps, raw["vocab_size"], 1900 + i) for i in range(100)]
    cfg, params = pm.read_model(folder, torch.float64)
    cfg_b, params_b = pm.read_model(folder, torch.bfloat16)
    ref, err = [], 0.0
    for p, f in zip(prompts, feeds):
        exact = pm.forward(cfg, params, p + f).numpy()[len(p):]
        rounded = pm.forward(cfg_b, params_b, p + f).float().numpy()[len(p):]
        ref.append(exact.astype(np.float32))
        err = max(err, float(np.abs(rounded - exact).max()))
    scale = max(float(np.abs(r).max()) for r in ref)
    return folder, raw, prompts, feeds, ref, scale, err / scale


@pytest.mark.parametrize("n_req", [12, 24, 40, 64, 100])
def test_decode_steps_of_9_to_128_requests(many_requests, n_req):
    """12 (at this width the products of gemm_mid.hip take a step from 9 rows on), 24, 40, 64 and 100 requests decode 12 steps side by side: eagerly and through captured graphs, every step's logits
    against each other and against the plain implementation.  The products must have run on the kernels of 17 to 128
    rows, the split ones added up by the norm that follows them."""
    from inferrs_amd.engine import Engine, Entry
    folder, raw, prompts, feeds, ref, scale, limit = many_requests
    n_steps = len(feeds[0])
    outs = {}
    for graphs in (False, True):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=n_req * 8, max_seqs=n_req + 1,
                                 use_graphs=graphs)
        for i in range(n_req):
            eng.step([Entry(i, prompts[i], [])])
        with CallCounter("gemm_mid_bf16", "add_rmsnorm_partials") as counted:
            rows = []
            for s in range(n_steps):
                logits = eng.step([Entry(i, [feeds[i][s]], [0]) for i in range(n_req)])
                rows.append(logits.cpu().numpy().copy())
                if s % 5 == 2:                   # an eager step of another shape between the replays
                    eng.step([Entry("extra", random_tokens(19, raw["vocab_size"], s), [18])])
                    eng.end_request("extra")
        outs[graphs] = rows
        assert (eng.graph_replays >= n_steps - 2) == graphs
        layers = raw["num_hidden_layers"]
        # q|k|v, o, [gate; up] and down of every layer in every step that was not a replay; o and down leave splits
        eager_steps = n_steps if not graphs else 2
        assert counted.calls["gemm_mid_bf16"] >= 4 * layers * eager_steps, counted.calls
        assert counted.calls["add_rmsnorm_partials"] >= (2 * layers - 1) * eager_steps, counted.calls
        eng.cache.check_invariants()
    for graphs in (False, True):
        for s in range(n_steps):
            want = np.stack([ref[i][s] for i in range(n_req)])
            err = float(np.abs(outs[graphs][s] - want).max()) / scale
            assert err <= limit, f"graphs={graphs} step {s}: {err:.3e} of the scale against the plain implementation ({limit:.3e})"
    # eager step and replay run the same kernels; the padded block tables may split the keys differently
    errs = [float(np.abs(outs[True][s] - outs[False][s]).max()) / scale for s in range(n_steps)]
    assert max(errs) <= limit / 2, f"replays differ from eager steps: {errs}"


@pytest.mark.parametrize("n_req", [24, 64])
def test_runs_of_decode_steps_of_many_requests(many_requests, n_req):
    """The generation loop queues eight decode steps of 24 or 64 requests at once; the tokens are those of single
    steps (greedy; both runs replay the same graphs, so the bits are the same)."""
    from inferrs_amd.engine import Engine, GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    folder, raw, prompts, *_ = many_requests
    results = {}
    for run in (1, 8):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=n_req * 8, max_seqs=n_req)
        loop = GenerationLoop(eng, decode_run=run, max_batch_size=n_req, stop_token_ids=[])
        reqs = [loop.add(prompts[i], SamplingParams.greedy(max_tokens=21)) for i in range(n_req)]
        with CallCounter("gemm_mid_bf16") as counted:
            loop.run()
        results[run] = [list(r.output) for r in reqs]
        assert counted.calls["gemm_mid_bf16"] > 0
        assert eng.graph_replays >= 12
        eng.cache.check_invariants()
        assert not eng.cache.sequences
    assert results[8] == results[1]
    assert all(len(o) == 21 for o in results[8])


def test_twenty_decodes_beside_a_prompt_portion(many_requests):
    """One step of 20 decoded tokens and a 30-token portion of another request's prompt (50 rows: the products of 17 to
    64 rows, the attention launched apart for the two kinds), against the plain implementation."""
    from inferrs_amd.engine import Engine, Entry
    folder, raw, prompts, feeds, ref, scale, limit = many_requests
    eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=200, max_seqs=22)
    for i in range(20):
        eng.step([Entry(i, prompts[i], [])])
    long = prompts[63] + feeds[63]
    cut = len(prompts[63]) - 25
    eng.step([Entry("p", long[:cut], [])])
    with CallCounter("gemm_mid_bf16") as counted:
        got = eng.step([Entry(i, [feeds[i][0]], [0]) for i in range(20)]
                       + [Entry("p", long[cut:cut + 30], [25, 29])]).cpu().numpy()
    assert counted.calls["gemm_mid_bf16"] >= 4 * raw["num_hidden_layers"]
    want = np.stack([ref[i][0] for i in range(20)] + [ref[63][0], ref[63][4]])
    err = float(np.abs(got - want).max()) / scale
    assert err <= limit, f"{err:.3e} of the scale against the plain implementation ({limit:.3e})"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "G"])
def test_logits_do_not_depend_on_where_the_pages_lie(models, tmp_path, name, dtype):
    """The same mixed trace over two pools: the smallest one that holds it, and a larger one whose free list was
    stirred first, so that every request's pages are other pages in another order.  Which pages hold a request's keys
    changes no arithmetic: the logits are the same bit for bit, in both precisions.  (Between two ways of cutting the
    work bfloat16 cannot be held tighter than against the plain implementation: each cutting rounds its own way, and
    the two differ from each other by 0.2 to 0.9 of the bound on these models, as either differs from the exact
    result by 0.4 to 0.8 of it.)"""
    from inferrs_amd.engine import Engine, run_trace
    folder, raw, reqs, ref = pick(models, name, True, dtype)
    trace = tm.mixed(reqs, seed=5)
    page = PAGE_SIZE[name]
    outs = []
    for extra in (0, 37):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page) + extra, max_seqs=4)
        if extra:
            pool = eng.cache.groups[0].pool
            taken = pool.allocate(pool.num_pages)
            pool.free(taken[1::2] + taken[0::2][::-1])          # odd pages first, then the even ones backwards
        out_dir = str(tmp_path / str(extra))
        run_trace(eng, trace.lines, out_dir, io.StringIO())
        eng.cache.check_invariants()
        outs.append(trace.read(out_dir, raw["vocab_size"]))
    for r, toks in reqs.items():
        for p in range(len(toks)):
            assert np.array_equal(outs[0][r][p], outs[1][r][p]), (r, p)
    err, where = worst(outs[1], ref, reqs)
    assert err <= bound(folder, reqs, ref, dtype), f"{err:.3e} at {where}"
