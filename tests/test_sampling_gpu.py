"""The device sampler against the plain transcription of the reference's sampler
(`tests/plain_model.py: sample`, from `inferrs/src/sampler.rs:146-335`), and the per-step random
number against the same transcription bit for bit."""
import math

import pytest
import torch

import plain_model as pm

from inferrs_amd.sampling import SamplingParams, rand_f32


def test_rand_f32_is_the_reference_function():
    for seed, step in [(0, 0), (1, 0), (42, 17), (2**63 + 5, 123456), (2**64 - 1, 2**40)]:
        assert rand_f32(seed, step) == pm.rand_f32(seed, step)
        assert 0.0 <= rand_f32(seed, step) <= 1.0
    draws = [rand_f32(7, s) for s in range(2000)]
    assert len(set(draws)) > 1990 and abs(sum(draws) / len(draws) - 0.5) < 0.03


def _case(vocab, seed, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(vocab, generator=g) * scale
    prev = torch.randint(0, vocab, (90,), generator=g).tolist()
    return z, prev


def _interval_of(z, prev, seed, token, kw):
    """In 64-bit: the stretch of the unit interval that the reference's walk gives `token`
    (inferrs/src/sampler.rs:186-335), and the random number of this draw."""
    z = z.double().clone()
    window = list(prev[-kw["repeat_last_n"]:]) if kw["repeat_last_n"] > 0 else []
    if kw["repetition_penalty"] not in (1.0, 0.0):
        for t in dict.fromkeys(window):
            z[t] = z[t] / kw["repetition_penalty"] if z[t] >= 0 else z[t] * kw["repetition_penalty"]
    for t in set(window):
        z[t] -= kw["frequency_penalty"] * window.count(t) + kw["presence_penalty"] if (kw["frequency_penalty"] or kw["presence_penalty"]) else 0.0
    p = torch.softmax(z / max(kw["temperature"], 1e-5), 0)
    order = sorted(range(len(p)), key=lambda i: (-float(p[i]), i))
    if 0 < kw["top_k"] < len(order):
        order = order[:kw["top_k"]]
    if kw["top_p"] < 1.0:
        cum = torch.cumsum(p[order], 0)
        cut = int((cum >= kw["top_p"]).nonzero()[0]) + 1 if bool((cum >= kw["top_p"]).any()) else len(order)
        order = order[:cut]
    if kw["min_p"] > 0.0:
        order = [i for i in order if float(p[i]) >= float(p[order[0]]) * kw["min_p"]] or order
    kept = p[order] / p[order].sum()
    cum = torch.cumsum(kept, 0)
    rank = order.index(token)
    return (float(cum[rank - 1]) if rank else 0.0), float(cum[rank]), rand_f32(seed, len(prev))


PARAMS = [
    dict(temperature=0.7, top_p=1.0, top_k=0, repetition_penalty=1.0),                 # plain tempered softmax
    dict(),                                                                            # the reference's defaults
    dict(temperature=1.3, top_p=0.5, top_k=0, repetition_penalty=1.0),
    dict(temperature=1.0, top_p=1.0, top_k=5, repetition_penalty=1.3, repeat_last_n=16),
    dict(temperature=0.9, top_p=0.95, top_k=40, min_p=0.2, frequency_penalty=0.4, presence_penalty=0.3),
    dict(temperature=2.0, top_p=1.0, top_k=0, min_p=0.05, repetition_penalty=1.0),
    dict(temperature=0.0, top_p=1.0, top_k=0, repetition_penalty=1.5),                 # greedy after penalties
    dict(temperature=0.8, top_k=1),
]


@pytest.mark.gpu
@pytest.mark.parametrize("vocab", [130, 387, 4097, 8193, 151936])      # one stretch of a row, two, three, and 38
@pytest.mark.parametrize("kw", PARAMS, ids=[str(i) for i in range(len(PARAMS))])
def test_sampler_matches_the_plain_transcription(vocab, kw):
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    rows, params, prevs, seeds, zs = 6, [], [], [], []
    for i in range(rows):
        z, prev = _case(vocab, 100 * len(zs) + i + 1000 * PARAMS.index(kw))
        zs.append(z)
        prevs.append(prev[: 3 + 17 * i])
        seeds.append(1000 + i)
        params.append(SamplingParams(seed=seeds[-1], **kw))
    logits = torch.stack(zs).to("cuda")
    before = logits.clone()
    got = sampler.sample(logits, params, prevs, seeds)
    assert torch.equal(logits, before), "the sampler must not change the caller's logits"
    for i in range(rows):
        if (vocab > 100000 and i > 1) or (vocab > 1000 and i > 3):
            continue                                   # the plain sampler is slow at large vocabularies
        full = {**dict(temperature=0.7, top_p=0.9, top_k=50, min_p=0.0, repetition_penalty=1.1, repeat_last_n=64,
                       frequency_penalty=0.0, presence_penalty=0.0), **kw}
        want = pm.sample(zs[i], prevs[i], seed=seeds[i], **full)
        if got[i] != want:
            # The reference walks its sorted list with a running 32-bit difference, the kernel with
            # tree sums: they may part where u falls within the rounding of those sums of a boundary.
            lo, hi, u = _interval_of(zs[i], prevs[i], seeds[i], got[i], full)
            assert lo - 2e-4 <= u <= hi + 2e-4, f"row {i}: device {got[i]} (interval {lo}..{hi}), plain {want}, u {u}"


@pytest.mark.gpu
@pytest.mark.parametrize("vocab,top_k", [(387, 1), (387, 50), (387, 386), (5000, 700), (151936, 50), (151936, 1024),
                                         (5000, 0), (151936, 0), (4097, 1024), (8193, 3), (12289, 1000), (12289, 0)])
def test_rows_with_a_top_k_take_the_same_tokens_on_both_paths(vocab, top_k):
    """Rows with a top_k up to 1,024 pick their top_k tokens out and walk them as the reference walks its sorted
    list; the other rows (and these, with the switch off) find the same prefixes by bisection over the keys.
    Rows without a top_k try the same with the first 1,024 tokens of their list and go the long way when neither
    the nucleus, nor the min_p cut, nor the walk ends within those (here: the rows with a high temperature)."""
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(vocab + top_k)
    rows = 24
    logits = (torch.randn(rows, vocab, generator=g) * 2.5).to(torch.bfloat16).float()      # coarse values: many ties
    temperature = torch.linspace(0.5, 1.5, rows)
    top_p = torch.tensor([1.0, 0.9, 0.6] * (rows // 3))
    min_p = torch.tensor([0.0, 0.0, 0.0, 0.1] * (rows // 4))
    u = torch.rand(rows, generator=g)
    k = torch.full((rows,), top_k, dtype=torch.int32)
    n_top = torch.full((rows,), 5, dtype=torch.int32)
    args = [t.to("cuda") for t in (logits, temperature, k, top_p, min_p, u, n_top)]
    fast = ops.sample(*args)
    ops.library().ia_sample_tune(0)
    try:
        slow = ops.sample(*args)
    finally:
        ops.library().ia_sample_tune(1)
    same = (fast[0] == slow[0]).cpu()
    # sequential sums there, tree sums here: a row may part where u lies within their rounding of a boundary
    assert int(same.sum()) >= rows - 1, (fast[0].tolist(), slow[0].tolist())
    assert torch.equal(fast[2].cpu()[same], slow[2].cpu()[same]), "the lists' first entries"
    lp_f, lp_s = fast[1].cpu()[same], slow[1].cpu()[same]
    finite = torch.isfinite(lp_s)
    assert torch.equal(torch.isfinite(lp_f), finite) and float((lp_f[finite] - lp_s[finite]).abs().max()) < 1e-4


@pytest.mark.gpu
def test_mixed_rows_do_not_influence_each_other():
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    z0, p0 = _case(387, 1)
    z1, p1 = _case(387, 2)
    a = SamplingParams(temperature=0.9, top_k=20, seed=5)
    b = SamplingParams.greedy()
    alone = sampler.sample(z0[None].to("cuda"), [a], [p0], [5])[0]
    both = sampler.sample(torch.stack([z1, z0]).to("cuda"), [b, a], [p1, p0], [0, 5])
    assert both == [int(torch.argmax(z1)), alone]


@pytest.mark.gpu
def test_equal_logits_are_taken_in_index_order():
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    z = torch.zeros(1, 64)
    z[0, 10:20] = 5.0                                   # ten equal favourites, the rest far below
    for step in range(40):
        p = SamplingParams(temperature=1.0, top_p=1.0, top_k=4, repetition_penalty=1.0, seed=3)
        prev = [0] * step
        got = sampler.sample(z.to("cuda"), [p], [prev], [3])[0]
        want = pm.sample(z[0], prev, temperature=1.0, top_p=1.0, top_k=4, repetition_penalty=1.0, seed=3)
        assert got == want and 10 <= got <= 13          # top-4 of ten equals: the first four by index


@pytest.mark.gpu
def test_equal_favourites_across_the_stretches_of_a_row_are_taken_in_index_order():
    """A row of 10,000 logits is the work of three blocks (stretches of 3,336 tokens), each of which leaves its own
    first top_k behind: eleven equal favourites that straddle the first border, and a row of nothing but equal
    logits, are still taken by ascending index over the whole row."""
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    z = torch.zeros(1, 10000)
    z[0, 3330:3341] = 6.0
    flat = torch.zeros(1, 10000)
    seen, seen_flat = set(), set()
    for step in range(60):
        p = SamplingParams(temperature=1.0, top_p=1.0, top_k=8, repetition_penalty=1.0, seed=11)
        prev = [0] * step
        got = sampler.sample(z.to("cuda"), [p], [prev], [11])[0]
        want = pm.sample(z[0], prev, temperature=1.0, top_p=1.0, top_k=8, repetition_penalty=1.0, seed=11)
        assert got == want and 3330 <= got <= 3337, (step, got, want)
        seen.add(got)
        got = sampler.sample(flat.to("cuda"), [p], [prev], [11])[0]
        assert got == pm.sample(flat[0], prev, temperature=1.0, top_p=1.0, top_k=8, repetition_penalty=1.0, seed=11)
        assert 0 <= got <= 7
        seen_flat.add(got)
    assert max(seen) >= 3336 and min(seen) < 3336, seen          # tokens on both sides of the border were drawn
    assert len(seen_flat) >= 5


@pytest.mark.gpu
def test_frequencies_follow_the_tempered_softmax():
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    z = torch.tensor([2.0, 1.0, 0.0, -1.0, 0.5, 1.5, -3.0, 0.2])
    temp = 0.7
    probs = torch.softmax(z / temp, 0)
    n = 4000
    p = SamplingParams(temperature=temp, top_p=1.0, top_k=0, repetition_penalty=1.0, seed=11)
    logits = z[None].repeat(n, 1).to("cuda")
    got = sampler.sample(logits, [p] * n, [[0] * s for s in range(n)], [11] * n)
    counts = torch.bincount(torch.tensor(got), minlength=8).float()
    chi2 = float(((counts - n * probs) ** 2 / (n * probs)).sum())
    assert chi2 < 24.3, f"chi-square {chi2:.1f} with 7 degrees of freedom (0.999 quantile is 24.3)"


# The reference's own penalty-window cases (inferrs/src/sampler.rs:606-704): logits, history, parameters, winner.
REFERENCE_CASES = [
    ([10.0, 8.0, 0.0, 0.0], [0, 1, 2, 3], dict(repetition_penalty=1.5, repeat_last_n=2), 0),    # 0 outside the window
    ([10.0, 8.0, 0.0, 0.0], [1, 2, 3, 0], dict(repetition_penalty=1.5, repeat_last_n=2), 1),    # 0 inside: 6.67 < 8
    ([10.0, 0.0, 0.0, 0.0], [0], dict(repetition_penalty=2.0, repeat_last_n=0), 0),             # window 0 disables
    ([10.0, 5.0], [0], dict(repetition_penalty=1.5, repeat_last_n=64), 0),                      # window beyond the history
    ([10.0, 5.0], [0], dict(repetition_penalty=10.0, repeat_last_n=64), 1),
    ([10.0, 5.0], [0], dict(repetition_penalty=0.0, repeat_last_n=64), 0),                      # 0.0 acts as disabled
]


@pytest.mark.parametrize("logits,history,kw,winner", REFERENCE_CASES)
def test_plain_sampler_on_the_reference_cases(logits, history, kw, winner):
    assert pm.sample(torch.tensor(logits), history, temperature=0.0, **kw) == winner


@pytest.mark.gpu
@pytest.mark.parametrize("logits,history,kw,winner", REFERENCE_CASES)
def test_device_sampler_on_the_reference_cases(logits, history, kw, winner):
    from inferrs_amd.sampling import Sampler
    got = Sampler("cuda:0").sample(torch.tensor([logits]).to("cuda"), [SamplingParams(temperature=0.0, seed=1, **kw)],
                                   [history], [1])
    assert got == [winner]


def test_the_arg_max_is_taken_only_where_the_reference_takes_it():
    """`sampler.rs:171-179`: a temperature under the threshold means the arg max of the untouched logits; with a penalty
    over a window that holds a token, a bias or log-probabilities the reference goes on and draws at the threshold."""
    eps = 1e-5
    plain = SamplingParams(temperature=0.0, repetition_penalty=1.0)
    assert plain.draw_temperature(0) == 0.0 and plain.draw_temperature(9) == 0.0
    pen = SamplingParams(temperature=0.0, repetition_penalty=1.1)
    assert pen.draw_temperature(0) == 0.0 and pen.draw_temperature(1) == eps          # an empty window changes nothing
    assert SamplingParams(temperature=0.0, repetition_penalty=1.1, repeat_last_n=0).draw_temperature(5) == 0.0
    assert SamplingParams(temperature=0.0, repetition_penalty=1.0, presence_penalty=0.5).draw_temperature(5) == eps
    assert SamplingParams(temperature=0.0, repetition_penalty=1.0, logit_bias={3: 1.0}).draw_temperature(0) == eps
    assert SamplingParams(temperature=0.0, repetition_penalty=1.0, logprobs=True).draw_temperature(0) == eps
    assert SamplingParams(temperature=0.7).draw_temperature(5) == 0.7


@pytest.mark.gpu
def test_equal_favourites_under_a_penalty_at_temperature_zero_are_drawn():
    """Two logits that are equal after a penalty touched the row, temperature 0: the reference does not take the arg max
    there but draws at a temperature of 1e-5, so either favourite comes, by the request's random number; a third
    that is 3e-5 below comes now and then too.  The device's draws are the plain transcription's, step by step, and
    both favourites occur."""
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    z = torch.randn(1, 5000, generator=torch.Generator().manual_seed(1))
    z[0, 1759] = z[0, 3155] = 7.0
    z[0, 77] = 7.0 - 3e-5
    kw = dict(temperature=0.0, top_p=1.0, top_k=1024, min_p=0.05, repetition_penalty=1.1, repeat_last_n=64,
              frequency_penalty=0.3, presence_penalty=0.2)
    seen = set()
    for step in range(3, 43):
        prev = [5, 6, 7] + [8] * (step - 3)
        got = sampler.sample(z.to("cuda"), [SamplingParams(seed=11, **kw)], [prev], [11])[0]
        assert got == pm.sample(z[0], prev, seed=11, **kw)
        seen.add(got)
    assert {1759, 3155} <= seen <= {1759, 3155, 77}
    # without a token in the window nothing touches the row: the arg max, the first of the equal ones
    assert sampler.sample(z.to("cuda"), [SamplingParams(seed=11, **kw)], [[]], [11]) == [1759]


@pytest.mark.gpu
@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_a_bias_on_the_logits_against_the_plain_transcription(temperature):
    """`sampler.rs:185-190`: the bias is added before the penalties; ids beyond the vocabulary are skipped; with a bias a
    temperature of 0 is no arg max of the raw logits (a bias that lifts a token to the top wins, one that makes two equal
    lets either come)."""
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    vocab = 3000
    z = torch.randn(vocab, generator=torch.Generator().manual_seed(4)) * 2
    top = int(torch.argmax(z))
    second = int(torch.topk(z, 2).indices[1])
    lift = {second: float(z[top] - z[second]) + 0.5, vocab + 7: 3.0}           # the second becomes the favourite
    level = {17: 9.0 - float(z[17]), 2500: 9.0 - float(z[2500])}               # two tokens made equal, above all others
    seen = set()
    for bias in (lift, level):
        for step in range(24):
            prev = [1, 2] + [3] * step
            kw = dict(temperature=temperature, top_p=0.95, top_k=40, repetition_penalty=1.2, repeat_last_n=16)
            got = sampler.sample(z[None].to("cuda"), [SamplingParams(seed=9, logit_bias=bias, **kw)], [prev], [9])[0]
            assert got == pm.sample(z, prev, seed=9, logit_bias=bias, **kw), (bias, step)
            if bias is level:
                seen.add(got)
            elif temperature == 0.0:
                assert got == second
    if temperature == 0.0:
        assert seen == {17, 2500}


def test_sampling_params_defaults_are_the_reference_defaults():
    # inferrs/src/sampler.rs:90-112 and its test at :586-603
    p = SamplingParams()
    assert (p.temperature, p.top_p, p.top_k, p.min_p) == (0.7, 0.9, 50, 0.0)
    assert (p.repetition_penalty, p.repeat_last_n, p.frequency_penalty, p.presence_penalty) == (1.1, 64, 0.0, 0.0)
    assert p.max_tokens == 2048 and p.seed is None and not p.bypass_stop_tokens
    with pytest.raises(ValueError):
        SamplingParams(top_p=0.0)


LOGPROB_PARAMS = [
    dict(temperature=0.7, top_p=1.0, top_k=0, repetition_penalty=1.0, top_logprobs=5),
    dict(top_logprobs=20),                                                   # the reference's defaults: top-k 50, top-p 0.9
    dict(temperature=1.0, top_p=1.0, top_k=3, repetition_penalty=1.3, repeat_last_n=16, top_logprobs=7),   # a list shorter than asked for
    dict(temperature=0.0, top_p=1.0, top_k=0, repetition_penalty=1.0, top_logprobs=4),    # greedy: no shortcut with log-probabilities
    dict(temperature=0.9, top_p=0.6, top_k=40, min_p=0.1, top_logprobs=0),
]


@pytest.mark.gpu
@pytest.mark.parametrize("vocab", [130, 2000, 151936])
@pytest.mark.parametrize("kw", LOGPROB_PARAMS, ids=[str(i) for i in range(len(LOGPROB_PARAMS))])
def test_log_probabilities_match_the_plain_transcription(vocab, kw):
    """`logprobs` (inferrs/src/sampler.rs:285-352): the drawn token's log-probability within the list that
    top-k, top-p and min-p kept, and the first `top_logprobs` entries of that list in its order."""
    from inferrs_amd.sampling import Sampler
    sampler = Sampler("cuda:0")
    rows = 4 if vocab < 100000 else 2
    zs, prevs, seeds, params = [], [], [], []
    for i in range(rows):
        z, prev = _case(vocab, 7000 + 10 * LOGPROB_PARAMS.index(kw) + i)
        zs.append(z); prevs.append(prev[: 5 + 11 * i]); seeds.append(50 + i)
        # a row without log-probabilities beside rows with them
        params.append(SamplingParams(seed=seeds[-1], logprobs=i != 1, **(kw if i != 1 else {k: v for k, v in kw.items() if k != "top_logprobs"})))
    tokens, infos = sampler.sample_with_logprobs(torch.stack(zs).to("cuda"), params, prevs, seeds)
    assert infos[1] is None
    full = {**dict(temperature=0.7, top_p=0.9, top_k=50, min_p=0.0, repetition_penalty=1.1, repeat_last_n=64,
                   frequency_penalty=0.0, presence_penalty=0.0), **kw}
    for i in range(rows):
        if i == 1:
            continue
        want_token, want_lp, want_top = pm.sample(zs[i], prevs[i], seed=seeds[i], logprobs=True, **full)
        info = infos[i]
        assert info.token_id == tokens[i]
        assert [t for t, _ in info.top_logprobs] == [t for t, _ in want_top]
        for (_, got), (_, want) in zip(info.top_logprobs, want_top):
            assert got == pytest.approx(want, abs=2e-3) or (math.isinf(got) and math.isinf(want))
        if tokens[i] == want_token:            # they may part where u falls on a boundary (see above)
            assert info.logprob == pytest.approx(want_lp, abs=2e-3) or (math.isinf(info.logprob) and math.isinf(want_lp))
        if kw.get("temperature") == 0.0:
            assert tokens[i] == int(torch.argmax(zs[i])) and info.logprob == pytest.approx(0.0, abs=1e-6)


def test_log_probability_parameters_are_checked():
    with pytest.raises(ValueError, match="needs logprobs"):
        SamplingParams(top_logprobs=3)
    with pytest.raises(ValueError, match="0..20"):
        SamplingParams(logprobs=True, top_logprobs=21)
    assert not SamplingParams.greedy(logprobs=True).is_plain_greedy and SamplingParams.greedy().is_plain_greedy


@pytest.mark.gpu
@pytest.mark.parametrize("w", [1, 5, 64, 100])
def test_window_push_alone(w):
    """A row's penalty window takes its new token: appended while the row's cap is not reached, else the oldest
    entry goes; rows without a window stay as they are.  Windows of up to 64 entries take a wave a row, wider
    ones a thread a row."""
    import torch
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(w)
    rows = 9
    caps = torch.tensor([0, 1, w, max(1, w // 2), w, w + 7, 2, w, 3], dtype=torch.int32)
    held = [0, 1, 0, max(1, w // 2), w, w, 1, max(0, w - 1), 0]
    window = torch.full((rows, w), -1, dtype=torch.int32)
    for r in range(rows):
        n = min(held[r], min(int(caps[r]), w))
        window[r, :n] = torch.randint(0, 1000, (n,), generator=g, dtype=torch.int32)
    tokens = torch.randint(0, 1000, (rows,), generator=g, dtype=torch.int32)
    want = window.clone()
    for r in range(rows):
        cap = min(int(caps[r]), w)
        if cap <= 0:
            continue
        have = int((want[r, :cap] >= 0).sum())
        if have < cap:
            want[r, have] = tokens[r]
        else:
            want[r, :cap - 1] = want[r, 1:cap].clone()
            want[r, cap - 1] = tokens[r]
    dev = "cuda:0"
    got = ops.window_push(window.to(dev), caps.to(dev), tokens.to(dev)).cpu()
    assert torch.equal(got, want)
