"""The serving loop under random settings: batch sizes, token budgets, prompt portions, runs of decode steps, row
multiples, page sizes and pools from the smallest that holds the longest request (requests are then put back and
started again) to one that holds them all.  Greedy generation in 32-bit must give the plain implementation's tokens
for every request whatever the settings, finish every request for its length, and leave every page free."""
import random

import pytest

import plain_model as pm
from tiny_configs import TINY, random_tokens, write_model

pytestmark = pytest.mark.gpu

NAMES = ("A", "B", "D", "G")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name in NAMES:
        folder = write_model(str(tmp_path_factory.mktemp(f"serve_{name}")), TINY[name], seed=3)
        out[name] = (folder,) + pm.read_model(folder)
    return out


@pytest.mark.parametrize("seed", range(6))
def test_random_settings_give_the_plain_tokens(folders, seed):
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    rng = random.Random(77 + seed)
    wanted = {}
    preempted = 0
    for case in range(8):
        name = rng.choice(NAMES)
        folder, cfg, params = folders[name]
        vocab = TINY[name]["vocab_size"]
        n_req = rng.choice([1, 2, 3, 5, 8, 12])
        prompts = [random_tokens(rng.choice([1, 2, 7, 20, 33, 64, 90]), vocab, rng.randrange(10 ** 6)) for _ in range(n_req)]
        n_new = [rng.choice([1, 2, 5, 12, 20]) for _ in range(n_req)]
        page = rng.choice([4, 8, 16])
        longest = -(-max(len(p) + n for p, n in zip(prompts, n_new)) // page)
        total = sum(-(-(len(p) + n) // page) for p, n in zip(prompts, n_new))
        pages = rng.choice([longest + 1, max(longest + 1, total // 2), total + 2])
        opts = dict(max_batch_size=rng.choice([1, 2, 4, 8, 16]), max_tokens_per_step=rng.choice([8, 16, 50, 256]),
                    prefill_chunk=rng.choice([None, 4, 16, 64]), decode_run=rng.choice([1, 3, 8]),
                    row_multiple=rng.choice([1, 8, 256]))
        what = f"configuration {name}, {n_req} requests, {pages} pages of {page}, {opts}"
        eng = Engine.from_folder(folder, dtype="float32", page_size=page, num_pages=pages, max_seqs=opts["max_batch_size"] + 1)
        outs = eng.generate(prompts, [SamplingParams.greedy(max_tokens=n, bypass_stop_tokens=True) for n in n_new], **opts)
        for prompt, n, out in zip(prompts, n_new, outs):
            key = (name, tuple(prompt), n)
            if key not in wanted:
                wanted[key] = pm.greedy(cfg, params, prompt, n)
            assert out.finish_reason == "length" and out.error is None, f"{what}: {out.finish_reason} {out.error}"
            assert out.tokens == wanted[key], what
            preempted += out.preemptions
        eng.cache.check_invariants()
        assert not eng.cache.sequences and all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups), what
    if seed == 0:
        assert preempted > 0, "no case of this seed ran out of pages: the smallest pools are meant to"


@pytest.mark.parametrize("seed", range(3))
def test_random_sampling_parameters_give_the_plain_chain(folders, seed):
    """The same with draws: every request with sampling parameters of its own (temperatures from 0 on, top-k, top-p,
    min-p, the three penalties over windows of 0, 4 or 64 tokens, now and then a bias on a few logits) and a seed, through
    single steps and runs of decode steps, beside up to ten others.  In 32-bit every token is the plain sampler's on the
    plain model's logits of the tokens so far (a draw within rounding of a boundary could part the chains; none of these does)."""
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    rng = random.Random(500 + seed)
    for case in range(6):
        name = rng.choice(("A", "B", "G"))
        folder, cfg, params = folders[name]
        vocab = TINY[name]["vocab_size"]
        n_req = rng.choice([1, 2, 4, 9, 11])
        prompts = [random_tokens(rng.choice([1, 3, 12, 40]), vocab, rng.randrange(10 ** 6)) for _ in range(n_req)]
        kws = []
        for _ in range(n_req):
            kw = dict(temperature=rng.choice([0.0, 0.0, 0.5, 1.0, 1.5]), top_p=rng.choice([1.0, 0.9, 0.5]),
                      top_k=rng.choice([0, 1, 5, 50]), min_p=rng.choice([0.0, 0.1]),
                      repetition_penalty=rng.choice([1.0, 1.1, 1.5]), repeat_last_n=rng.choice([0, 4, 64]),
                      frequency_penalty=rng.choice([0.0, 0.4]), presence_penalty=rng.choice([0.0, 0.3]))
            if rng.random() < 0.3:
                kw["logit_bias"] = {rng.randrange(vocab): rng.choice([-5.0, 2.0, 8.0]) for _ in range(rng.choice([1, 3]))}
            kws.append(kw)
        seeds = [rng.randrange(10 ** 6) for _ in range(n_req)]
        n_new = rng.choice([3, 9, 20])
        opts = dict(max_batch_size=rng.choice([2, 4, 16]), max_tokens_per_step=rng.choice([16, 64, 256]),
                    decode_run=rng.choice([1, 4, 8]))
        eng = Engine.from_folder(folder, dtype="float32", page_size=rng.choice([4, 16]), num_pages=400, max_seqs=17)
        outs = eng.generate(prompts, [SamplingParams(seed=s, max_tokens=n_new, bypass_stop_tokens=True, **kw)
                                      for s, kw in zip(seeds, kws)], **opts)
        for i, out in enumerate(outs):
            toks = list(prompts[i])
            for j in range(n_new):
                want = pm.sample(pm.forward(cfg, params, toks)[-1].float(), toks, seed=seeds[i], **kws[i])
                assert out.tokens[j] == want, f"case {case}, configuration {name}, request {i}, token {j}: {kws[i]} {opts}"
                toks.append(want)
        eng.cache.check_invariants()
        assert not eng.cache.sequences
