"""Generation through the entry points: the Python one (`Engine.generate`), the scheduler under
a tight pool, and the command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_model as pm
from tiny_configs import TINY, random_tokens, write_model

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    out = {}
    for name in ("A", "B"):
        folder = write_model(str(tmp_path_factory.mktemp(f"gen_{name}")), TINY[name], seed=21)
        out[name] = (folder, *pm.read_model(folder, torch.float64))
    return out


def plain_greedy_with_margins(cfg, params, prompt, n):
    """Greedy continuation and, per step, the gap between the best and the second logit."""
    toks, margins = list(prompt), []
    for _ in range(n):
        row = pm.forward(cfg, params, toks)[-1]
        top = torch.topk(row, 2).values
        margins.append(float(top[0] - top[1]))
        toks.append(int(torch.argmax(row)))
    return toks[len(prompt):], margins


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("A", "bfloat16"), ("B", "bfloat16")])
def test_greedy_generation_matches_plain(tiny, name, dtype):
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny[name]
    vocab = TINY[name]["vocab_size"]
    prompts = [random_tokens(n, vocab, 50 + n) for n in (5, 17, 33, 1)]       # prompts of 5, 17 and 33 tokens with 16 greedy tokens each, and a prompt of one token
    eng = Engine.from_folder(folder, dtype=dtype, page_size=4, num_pages=64, max_seqs=4)
    outs = eng.generate(prompts, SamplingParams.greedy(max_tokens=16), max_tokens_per_step=24, prefill_chunk=16)
    for prompt, out in zip(prompts, outs):
        want, margins = plain_greedy_with_margins(cfg, params, prompt, 16)
        assert out.finish_reason == "length" and len(out.tokens) == 16
        if dtype == "float32":
            assert out.tokens == want
        else:
            # bfloat16 may legitimately differ where two logits are closer than its rounding; up to there it agrees
            for i, (g, w) in enumerate(zip(out.tokens, want)):
                if g != w:
                    assert margins[i] < 0.02, f"token {i}: {g} != {w} with a margin of {margins[i]:.3f}"
                    break
    eng.cache.check_invariants()
    assert not eng.cache.sequences


def test_seeded_temperature_is_reproducible_and_independent_of_the_batch(tiny):
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["B"]
    vocab = TINY["B"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 70 + n) for n in (1, 9, 64, 100)]      # prompts of 1, 9, 64 and 100 tokens at temperature 0.7 under fixed seeds, portions of 16
    sp = [SamplingParams(temperature=0.7, top_p=1.0, top_k=0, repetition_penalty=1.0, max_tokens=12, seed=40 + i)
          for i in range(4)]
    eng = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=64, max_seqs=4)
    together = eng.generate(prompts, sp, prefill_chunk=16)
    alone = [eng.generate([p], [s])[0] for p, s in zip(prompts, sp)]
    assert [g.tokens for g in together] == [g.tokens for g in alone]
    # and each token is what the plain sampler draws from the plain model's logits
    toks = list(prompts[1])
    for t in together[1].tokens:
        row = pm.forward(cfg, params, toks)[-1].float()
        assert t == pm.sample(row, toks, temperature=0.7, top_p=1.0, top_k=0, repetition_penalty=1.0, seed=41)
        toks.append(t)


def test_tight_pool_preempts_and_still_gives_the_same_tokens(tiny):
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["A"]
    vocab = TINY["A"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 90 + n) for n in (20, 24, 28, 18)]
    sp = SamplingParams.greedy(max_tokens=24)
    roomy = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=256, max_seqs=4)
    want = roomy.generate(prompts, sp)
    tight = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=30, max_seqs=4)    # 120 slots for ~186 tokens
    got = tight.generate(prompts, sp)
    assert sum(g.preemptions for g in got) > 0 and sum(g.preemptions for g in want) == 0
    assert [g.tokens for g in got] == [g.tokens for g in want]
    assert all(g.finish_reason == "length" for g in got)
    tight.cache.check_invariants()
    too_small = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=5, max_seqs=4)
    res = too_small.generate([prompts[0], prompts[0][:6]], SamplingParams.greedy(max_tokens=4))
    assert res[0].finish_reason == "error" and "out of KV blocks" in res[0].error
    assert res[1].finish_reason == "length" and len(res[1].tokens) == 4


def test_stop_token_ends_generation(tiny):
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["A"]
    prompt = random_tokens(9, TINY["A"]["vocab_size"], 5)
    want, _ = plain_greedy_with_margins(cfg, params, prompt, 6)
    eng = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=64, max_seqs=2)
    out = eng.generate([prompt], SamplingParams.greedy(max_tokens=6, extra_stop_token_ids=(want[2],)))[0]
    first = want.index(want[2])
    assert out.tokens == want[:first + 1] and out.finish_reason == "stop"
    out = eng.generate([prompt], SamplingParams.greedy(max_tokens=6, extra_stop_token_ids=(want[2],),
                                                       bypass_stop_tokens=True))[0]
    assert out.tokens == want and out.finish_reason == "length"


def test_command_line_run_and_bench(tiny):
    folder, cfg, params = tiny["A"]
    prompt = random_tokens(7, TINY["A"]["vocab_size"], 3)
    want, _ = plain_greedy_with_margins(cfg, params, prompt, 5)
    exe = [sys.executable, os.path.join(ROOT, "bin", "inferrs-amd")]
    proc = subprocess.run(exe + ["run", folder, ",".join(map(str, prompt)), "--dtype", "f32", "--temperature", "0",
                                 "--repetition-penalty", "1.0", "--max-tokens", "5", "--block-size", "4",
                                 "--max-blocks", "32", "--max-batch-size", "2"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == want
    assert "finish: length" in proc.stderr
    proc = subprocess.run(exe + ["bench", folder, "--dtype", "bf16", "--prompt-len", "32", "--max-tokens", "8",
                                 "--runs", "2", "--max-blocks", "32", "--max-batch-size", "2"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().splitlines()[-1])
    assert rec["prefill_tok_s"] > 0 and rec["decode_tok_s"] > 0
    # without a prompt: one prompt a line from standard input, each answered on its own
    other = random_tokens(4, TINY["A"]["vocab_size"], 8)
    want_other, _ = plain_greedy_with_margins(cfg, params, other, 5)
    script = " ".join(map(str, prompt)) + "\n\n" + ",".join(map(str, other)) + "\n"
    proc = subprocess.run(exe + ["run", folder, "--dtype", "f32", "--temperature", "0", "--repetition-penalty", "1.0",
                                 "--max-tokens", "5", "--block-size", "4", "--max-blocks", "32", "--max-batch-size", "2"],
                          input=script, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = proc.stdout.splitlines()
    assert [[int(t) for t in line.split()] for line in out] == [want, want_other]
    proc = subprocess.run(exe + ["serve", folder], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 2 and "not part of this engine" in proc.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_runs_of_decode_steps_give_the_same_tokens_as_single_steps(tiny, dtype):
    """Greedy requests decode several steps at a time once their shape is captured; the tokens,
    the stop at a stop token in the middle of a run and the end at max_tokens are those of
    single steps."""
    from inferrs_amd.engine import Engine, GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["B"]
    vocab = TINY["B"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 300 + n) for n in (7, 30, 12)]
    results = {}
    for run in (1, 8):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=64, max_seqs=4)
        loop = GenerationLoop(eng, decode_run=run)
        stop = None if run == 1 else results[1][0][20]           # a token that request 0 emits on its way
        sp = [SamplingParams.greedy(max_tokens=40, extra_stop_token_ids=() if i or stop is None else (stop,))
              for i in range(3)]
        sp[2] = SamplingParams.greedy(max_tokens=23)
        reqs = [loop.add(p, s) for p, s in zip(prompts, sp)]
        loop.run()
        results[run] = [list(r.output) for r in reqs]
        if run == 8:
            assert eng.graph_replays > 10
            assert reqs[0].finish_reason == "stop" and reqs[1].finish_reason == reqs[2].finish_reason == "length"
        eng.cache.check_invariants()
        assert not eng.cache.sequences
    first = results[1][0].index(results[1][0][20])
    assert results[8][0] == results[1][0][:first + 1]
    assert results[8][1] == results[1][1] and results[8][2] == results[1][2] and len(results[8][2]) == 23


def test_runs_of_decode_steps_draw_the_same_tokens_as_single_steps(tiny):
    """Requests that draw (temperature, top-k, top-p, min-p, penalties over a window that fills up and then
    moves, a logit bias; a greedy one with a penalty among them) also decode several steps at a time: the
    random numbers of the run and the penalty windows live on the device, and the tokens are those of
    single steps."""
    from inferrs_amd.engine import Engine, GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, params = tiny["B"]
    vocab = TINY["B"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 500 + n) for n in (7, 30, 12, 3)]
    sps = [SamplingParams(seed=11, max_tokens=45),                                           # the reference's defaults
           SamplingParams(seed=12, max_tokens=45, temperature=1.2, top_k=0, top_p=0.8, repetition_penalty=1.0,
                          frequency_penalty=0.3, presence_penalty=0.2, repeat_last_n=9),
           SamplingParams(seed=13, max_tokens=31, temperature=0.0, repetition_penalty=1.4, repeat_last_n=20),
           SamplingParams(seed=14, max_tokens=45, temperature=0.9, top_k=12, min_p=0.05, repetition_penalty=1.0,
                          logit_bias={5: 2.0, 17: -3.0})]
    results = {}
    for run in (1, 8):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=64, max_seqs=5)
        loop = GenerationLoop(eng, decode_run=run, stop_token_ids=[])
        reqs = [loop.add(p, s) for p, s in zip(prompts, sps)]
        loop.run()
        results[run] = [list(r.output) for r in reqs]
        if run == 8:
            assert eng.graph_replays > 20
        eng.cache.check_invariants()
        assert not eng.cache.sequences
    assert results[8] == results[1]
    assert [len(o) for o in results[8]] == [45, 45, 31, 45]


def test_generation_reports_log_probabilities(tiny):
    """`logprobs` through the entry point: one record per generated token, consistent with the plain
    model's softmax at that place (temperature 1, nothing filtered, so the kept list is the vocabulary)."""
    import math
    from inferrs_amd import SamplingParams
    from inferrs_amd.engine import Engine
    folder, cfg, params = tiny["B"]
    eng = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=40, max_seqs=4)
    prompt = random_tokens(9, cfg["vocab_size"], 71)
    sp = SamplingParams(temperature=1.0, top_p=1.0, top_k=0, repetition_penalty=1.0, seed=3, max_tokens=6,
                        logprobs=True, top_logprobs=4, bypass_stop_tokens=True)
    plain = SamplingParams(temperature=1.0, top_p=1.0, top_k=0, repetition_penalty=1.0, seed=3, max_tokens=6,
                           bypass_stop_tokens=True)
    with_lp, without = eng.generate([prompt, prompt], [sp, plain])
    assert with_lp.tokens == without.tokens and without.logprobs is None      # asking for them changes no draw
    assert len(with_lp.logprobs) == 6
    toks = list(prompt)
    for tok, info in zip(with_lp.tokens, with_lp.logprobs):
        logp = torch.log_softmax(pm.forward(cfg, params, toks)[-1], 0)
        assert info.token_id == tok and info.logprob == pytest.approx(float(logp[tok]), abs=1e-4)
        best = torch.topk(logp, 4)
        assert [t for t, _ in info.top_logprobs] == best.indices.tolist()
        assert [v for _, v in info.top_logprobs] == pytest.approx(best.values.tolist(), abs=1e-4)
        toks.append(tok)


def test_stop_strings_and_cancellation(tiny):
    """`stop_strings` (`check_stop`, inferrs/src/engine.rs:866-887): generation ends with "stop" as soon as the
    decoded output ends with one of them; a request can also be cancelled between steps."""
    from inferrs_amd import SamplingParams
    from inferrs_amd.engine import Engine, GenerationLoop
    folder, cfg, params = tiny["A"]
    eng = Engine.from_folder(folder, dtype="float32", page_size=4, num_pages=64, max_seqs=4)
    prompt = random_tokens(7, cfg["vocab_size"], 5)
    free = eng.generate([prompt], SamplingParams.greedy(max_tokens=12, bypass_stop_tokens=True))[0].tokens
    words = lambda ids: "".join(f"<{t}>" for t in ids)                     # a stand-in for a tokenizer
    stop = f"<{free[4]}><{free[5]}>"                                       # two tokens long: matched across tokens
    cut = next(i for i in range(1, 12) if words(free[:i + 1]).endswith(stop))
    sp = SamplingParams.greedy(max_tokens=12, bypass_stop_tokens=True, stop_strings=("", "never", stop))
    out = eng.generate([prompt, prompt], [sp, SamplingParams.greedy(max_tokens=12, bypass_stop_tokens=True)],
                       detokenize=words)
    assert out[0].tokens == free[:cut + 1] and out[0].finish_reason == "stop"
    assert out[1].tokens == free and out[1].finish_reason == "length"
    # a stop string at the very last allowed token still reads "stop"
    last = eng.generate([prompt], SamplingParams.greedy(max_tokens=cut + 1, bypass_stop_tokens=True, stop_strings=(stop,)),
                        detokenize=words)[0]
    assert last.tokens == free[:cut + 1] and last.finish_reason == "stop"
    with pytest.raises(ValueError, match="detokenizer"):
        eng.generate([prompt], sp)
    # cancellation
    loop = GenerationLoop(eng)
    a = loop.add(prompt, SamplingParams.greedy(max_tokens=50, bypass_stop_tokens=True))
    b = loop.add(prompt, SamplingParams.greedy(max_tokens=6, bypass_stop_tokens=True))
    loop.step()
    loop.step()
    loop.cancel(a)
    loop.run()
    assert a.finish_reason == "cancelled" and 0 < len(a.output) < 50 and b.output == free[:6]
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
