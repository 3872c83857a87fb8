"""Random tiny configurations of the architecture through the engine against the plain implementation: head sizes in
and out of the steps of 16 (8 to 256), any number of heads and groups, widths, feed-forward sizes and vocabularies that
are odd or no power of two, one to three layers, several eps and theta, page sizes from 4 to 48.  Every case runs three
requests whole and mixed (portions of some beside decoded tokens of others, in a pool that makes pages come back), in
32-bit and bfloat16.  A size is either computed right or refused with an error that names it; none is refused today."""
import io
import random

import numpy as np
import pytest
import torch

import plain_model as pm
import trace_modes as tm
from tiny_configs import random_tokens, write_model

pytestmark = pytest.mark.gpu

CASES = 40


def draw(case: int):
    rng = random.Random(1000 + case)
    nkv = rng.choice([1, 2, 3, 4, 5])
    g = rng.choice([1, 2, 3, 4, 5, 7, 8])
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3",
               vocab_size=rng.choice([61, 100, 257, 301, 1000, 1023, 4097, 9001]),
               hidden_size=rng.choice([32, 33, 34, 40, 50, 66, 70, 72, 77, 90, 98, 100, 130, 136, 200, 250, 262]),
               intermediate_size=rng.choice([32, 47, 50, 80, 94, 110, 150, 161, 256, 300, 386]),
               num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=nkv * g, num_key_value_heads=nkv,
               head_dim=rng.choice([8, 16, 24, 32, 40, 48, 64, 80, 96, 112, 128, 144, 256]),
               rope_theta=rng.choice([10000.0, 1e6, 500000.0]), rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-4]),
               tie_word_embeddings=rng.choice([True, False]), max_position_embeddings=512)
    page = rng.choice([4, 8, 16, 32, 48])
    lengths = [rng.choice([3, 9, 33]), rng.choice([40, 70]), rng.choice([100, 150])]
    return raw, page, lengths


@pytest.mark.parametrize("case", range(CASES))
def test_a_random_configuration_matches_plain(tmp_path, case):
    from inferrs_amd.engine import Engine, run_trace
    raw, page, lengths = draw(case)
    what = (f"head size {raw['head_dim']}, heads {raw['num_attention_heads']}/{raw['num_key_value_heads']}, width "
            f"{raw['hidden_size']}, feed-forward {raw['intermediate_size']}, vocabulary {raw['vocab_size']}, "
            f"{raw['num_hidden_layers']} layers, pages of {page}")
    folder = write_model(str(tmp_path / "m"), raw, seed=case)
    cfg, params = pm.read_model(folder, torch.float64)
    reqs = {f"r{i}": random_tokens(n, raw["vocab_size"], 10 * case + i) for i, n in enumerate(lengths)}
    ref = {r: pm.forward(cfg, params, t).numpy().astype(np.float32) for r, t in reqs.items()}
    scale = max(float(np.abs(v).max()) for v in ref.values())
    cfg16, p16 = pm.read_model(folder, torch.bfloat16)
    bf16_bound = max(float(np.abs(pm.forward(cfg16, p16, t).float().numpy() - ref[r]).max()) for r, t in reqs.items()) / scale
    for dtype, allowed in (("float32", 1e-5), ("bfloat16", bf16_bound)):
        for mode, trace in (("whole", tm.whole(reqs)), ("mixed", tm.mixed(reqs, seed=case, max_live=3, decode_tail=12))):
            eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page), max_seqs=4)
            out = str(tmp_path / f"{dtype}_{mode}")
            run_trace(eng, trace.lines, out, io.StringIO())
            eng.cache.check_invariants()
            got = trace.read(out, raw["vocab_size"])
            worst = max(float(np.abs(got[r][p] - ref[r][p]).max()) for r, t in reqs.items() for p in range(len(t))) / scale
            assert worst <= allowed, f"{what}; {dtype}, {mode}: {worst:.3e} of the largest logit (allowed {allowed:.3e})"
