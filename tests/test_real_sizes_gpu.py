"""The engine at the layer sizes of real models (Qwen3-8B: width 4,096, 32 query and 8 key/value heads of 128,
feed-forward 12,288; Qwen3-14B: width 5,120, 40 query heads, feed-forward 17,408, a width that is no power of two;
Qwen3-0.6B: width 1,024 under 16 heads of 128, so that the heads are twice as wide as the stream, the head tied to the
table; Qwen3-4B: width 2,560, feed-forward 9,728; Qwen3-32B: 64 query heads, feed-forward 25,600, whose [gate; up] is past what
the kernel with the activation inside takes at 17 to 64 rows;
two layers each and a vocabulary of 40,000 so that the plain implementation stays quick) against the
plain implementation in 64-bit: a prompt of 300 tokens whole and then token by token, 24 short requests decoded together, the last of them beside the two portions of another request's prompt,
and (8B sizes) a prompt of 2,600 tokens in portions of 1,024 with tokens decoded behind it, and 40 tokens decoded from a
context of 1,000 on.  The tiny configurations reach every code path; this one runs the shapes that the
size rules of the kernels pick at these widths (the skinny products with the stream inside up to 8 rows, the
products of 9 to 128 rows with their split sums, the vendor's products beyond, [gate; up] on 256 blocks, the decode
attention's splits, the tiled prompt attention, the 32-bit products' block shapes), whole steps of them together.

Tolerances as in the replay tests: 32-bit 1e-5 of the largest logit; bfloat16 the bound measured on this model (the
plain implementation in bfloat16 tensor arithmetic against itself in 64-bit)."""
import json
import os

import numpy as np
import pytest
import torch

import plain_model as pm
from tiny_configs import random_tokens

pytestmark = pytest.mark.gpu

RAW = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=40000, hidden_size=4096,
           intermediate_size=12288, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
           rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)
SHAPES = {"8B": RAW, "14B": dict(RAW, hidden_size=5120, intermediate_size=17408, num_attention_heads=40),
          "0.6B": dict(RAW, hidden_size=1024, intermediate_size=3072, num_attention_heads=16, tie_word_embeddings=True),
          "4B": dict(RAW, hidden_size=2560, intermediate_size=9728, tie_word_embeddings=True),
          "32B": dict(RAW, hidden_size=5120, intermediate_size=25600, num_attention_heads=64)}
PROMPT, DECODED = 300, 24          # one long request: its prompt whole, then token by token
CROWD, CROWD_PROMPT = 24, 30       # many short requests: their prompts in one step, then decoded together
FAR, FAR_PORTION, FAR_DECODED = 2600, 1024, 6     # a request with a context of thousands: its prompt in portions, then token by token
CROSS, CROSS_DECODED = 1000, 40    # a request whose decoded tokens pass a context of 1,024: another captured graph, another split of the keys
MIX, MIX_PORTION = 260, 150        # a request whose prompt comes in two portions beside the last eight decoding requests


@pytest.fixture(scope="module", params=sorted(SHAPES))
def real(request, tmp_path_factory):
    """The model's folder (weights drawn on the GPU: the host's generator takes minutes at this size), the requests
    and their 64-bit logits."""
    from inferrs_amd.config import Qwen3Config
    from inferrs_amd.parts import generated_tensors
    from inferrs_amd.weights import random_tensors, write_safetensors
    folder = str(tmp_path_factory.mktemp("real_sizes"))
    config = Qwen3Config.from_dict(SHAPES[request.param])
    tensors = random_tensors(generated_tensors(config.to_spec()), 3, torch.bfloat16, device="cuda:0")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f)
    write_safetensors(os.path.join(folder, "model.safetensors"), {k: v.cpu() for k, v in tensors.items()})
    del tensors
    torch.cuda.empty_cache()
    cfg, params = pm.read_model(folder, torch.float64)
    reqs = {"long": random_tokens(PROMPT + DECODED, RAW["vocab_size"], 50)}
    for i in range(CROWD):
        reqs[f"c{i}"] = random_tokens(CROWD_PROMPT + 3 * i % 7 + 12, RAW["vocab_size"], 60 + i)
    reqs["mix"] = random_tokens(MIX, RAW["vocab_size"], 53)
    if request.param == "8B":
        reqs["far"] = random_tokens(FAR + FAR_DECODED, RAW["vocab_size"], 51)
        reqs["cross"] = random_tokens(CROSS + CROSS_DECODED, RAW["vocab_size"], 52)
    ref = {}
    for r, t in reqs.items():
        full = pm.forward(cfg, params, t)
        if r == "far":            # (only the rows that the engine is asked for: the others would be 400 MB)
            keep = sorted({lo for lo in range(0, FAR, FAR_PORTION)} | {min(FAR, lo + FAR_PORTION) - 1 for lo in range(0, FAR, FAR_PORTION)}
                          | set(range(FAR, FAR + FAR_DECODED)))
            ref[r] = {p: full[p].numpy().astype(np.float32) for p in keep}
        else:
            ref[r] = full.numpy().astype(np.float32)
        del full
    del params
    cfg16, p16 = pm.read_model(folder, torch.bfloat16)
    rounded = pm.forward(cfg16, p16, reqs["long"]).float().numpy()
    scale = max(float(np.abs(v).max()) for r, v in ref.items() if r != "far")
    bf16_bound = float(np.abs(rounded - ref["long"]).max()) / scale
    return folder, reqs, ref, scale, bf16_bound


def run(folder, reqs, dtype):
    """{request: {position: logits}} of the long request (prompt whole, then single tokens) and of the crowd (prompts
    in one step, then decode steps of 24, 12 and 8 requests), the next token always the request's own next one."""
    from inferrs_amd.engine import Engine, Entry
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=200, max_seqs=CROWD + 2)
    got = {r: {} for r in reqs}
    if "far" in reqs:
        toks = reqs["far"]
        for lo in range(0, FAR, FAR_PORTION):
            hi = min(FAR, lo + FAR_PORTION)
            rows = eng.step([Entry("far", toks[lo:hi], [0, hi - lo - 1])]).cpu().numpy()      # a portion's first and last token
            got["far"][lo], got["far"][hi - 1] = rows[0], rows[1]
        for p in range(FAR, FAR + FAR_DECODED):
            got["far"][p] = eng.step([Entry("far", [toks[p]], [0])])[0].cpu().numpy()
        eng.end_request("far")
        toks = reqs["cross"]
        got["cross"][CROSS - 1] = eng.step([Entry("cross", toks[:CROSS], [CROSS - 1])])[0].cpu().numpy()
        for p in range(CROSS, CROSS + CROSS_DECODED):
            got["cross"][p] = eng.step([Entry("cross", [toks[p]], [0])])[0].cpu().numpy()
        eng.end_request("cross")
    toks = reqs["long"]
    got["long"][PROMPT - 1] = eng.step([Entry("long", toks[:PROMPT], [PROMPT - 1])])[0].cpu().numpy()
    for p in range(PROMPT, PROMPT + DECODED):
        got["long"][p] = eng.step([Entry("long", [toks[p]], [0])])[0].cpu().numpy()
    eng.end_request("long")
    crowd = [r for r in reqs if r.startswith("c")]
    rows = eng.step([Entry(r, reqs[r][:CROWD_PROMPT], [CROWD_PROMPT - 1]) for r in crowd]).cpu().numpy()
    for r, row in zip(crowd, rows):
        got[r][CROWD_PROMPT - 1] = row
    at = {r: CROWD_PROMPT for r in crowd}
    live = list(crowd)
    for step in range(12):
        live = [r for r in live if at[r] < len(reqs[r])]
        if step == 4:
            for r in live[12:]:
                eng.end_request(r)
            live = live[:12]
        if step == 8:
            for r in live[8:]:
                eng.end_request(r)
            live = live[:8]
        if not live:
            break
        rows = eng.step([Entry(r, [reqs[r][at[r]]], [0]) for r in live]).cpu().numpy()
        for r, row in zip(live, rows):
            got[r][at[r]] = row
            at[r] += 1
    # two mixed steps: the decoding requests that are left beside a portion of another request's prompt
    for lo, hi in ((0, MIX_PORTION), (MIX_PORTION, MIX)):
        live = [r for r in live if at[r] < len(reqs[r])]
        rows = eng.step([Entry("mix", reqs["mix"][lo:hi], [0, hi - lo - 1])] + [Entry(r, [reqs[r][at[r]]], [0]) for r in live]).cpu().numpy()
        got["mix"][lo], got["mix"][hi - 1] = rows[0], rows[1]
        for r, row in zip(live, rows[2:]):
            got[r][at[r]] = row
            at[r] += 1
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes_match_plain(real, dtype):
    folder, reqs, ref, scale, bf16_bound = real
    got = run(folder, reqs, dtype)
    allowed = 1e-5 if dtype == "float32" else bf16_bound
    assert sum(len(v) for v in got.values()) >= 1 + DECODED + CROWD + 4 * CROWD + 4 * 12 - 40
    worst, where = 0.0, None
    for r, rows in got.items():
        for p, row in rows.items():
            e = float(np.abs(row - ref[r][p]).max()) / scale
            if not e <= worst:
                worst, where = e, (r, p)
    print(f"real layer sizes, {dtype}: worst difference {worst:.3e} of the largest logit ({scale:.2f}) at {where}, allowed {allowed:.3e}")
    assert worst <= allowed, f"{dtype}: {worst:.3e} of the largest logit at {where} (allowed {allowed:.3e})"
    # and the greedy choice agrees wherever the plain model's first two candidates are further apart than the bound
    for r, rows in got.items():
        for p, row in rows.items():
            top2 = np.sort(ref[r][p])[-2:]
            if top2[1] - top2[0] > 2 * allowed * scale:
                assert int(np.argmax(row)) == int(np.argmax(ref[r][p])), (r, p)
