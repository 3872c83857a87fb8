"""Pins the plain implementation by what fixes it beside the reference's text: the reference's
own test vectors, special cases that reduce to a library routine, and invariants, each chosen
so that a plausible mistake (a sign, a pairing, a norm in the wrong place) fails it."""
import math

import pytest
import torch

import plain_model as pm
from tiny_configs import TINY, random_tokens, write_model


def test_rms_norm_reference_vector():
    # candle-nn/tests/ops.rs:55-66
    x = torch.tensor([[[3., 1., 4.], [1., 5., 9.]], [[2., 1., 7.], [8., 2., 8.]]])
    w = torch.tensor([1., 2., 3.])
    got = pm.rms_norm(x, w, 1e-5)
    want = torch.tensor([[[1.019, 0.6794, 4.0762], [0.1674, 1.6744, 4.521]],
                         [[0.4714, 0.4714, 4.9497], [1.206, 0.603, 3.6181]]])
    assert torch.equal(torch.round(got * 1e4) / 1e4, want)


def test_rms_norm_invariants():
    torch.manual_seed(0)
    x = torch.randn(5, 70, dtype=torch.float64)
    ones = torch.ones(70, dtype=torch.float64)
    y = pm.rms_norm(x, ones, 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(pm.rms_norm(3.7 * x, ones, 0.0), y, atol=1e-12)       # scale invariance
    # eps sits inside the root, added to the MEAN of squares (not the sum, not outside)
    v = torch.tensor([[2.0, 0.0, 0.0, 0.0]], dtype=torch.float64)
    assert math.isclose(pm.rms_norm(v, torch.ones(4, dtype=torch.float64), 3.0)[0, 0].item(), 2.0 / 2.0)


def test_softmax_reference_vectors():
    # candle-nn/tests/ops.rs:9-53 (last dimension) and :149-156
    x = torch.tensor([[[3., 1., 4.], [1., 5., 9.]], [[2., 1., 7.], [8., 2., 8.]]])
    got = pm.softmax_last(torch.log(x))
    want = torch.tensor([[[0.375, 0.125, 0.5], [0.0667, 0.3333, 0.6]],
                         [[0.2, 0.1, 0.7], [0.4444, 0.1111, 0.4444]]])
    assert torch.equal(torch.round(got * 1e4) / 1e4, want)
    assert pm.softmax_last(torch.tensor([1234., 0.])).tolist() == [1.0, 0.0]


def test_linear_reference_example():
    # candle-nn/src/linear.rs:7-20
    w = torch.tensor([[1., 2.], [3., 4.], [5., 6.]])
    assert pm.linear(torch.tensor([[10., 100.]]), w).tolist() == [[210., 430., 650.]]


def test_inv_freq():
    f = pm.inv_freq(1e6, 32)
    assert f[0].item() == 1.0
    want = torch.tensor([1e6 ** (-2 * i / 32) for i in range(16)], dtype=torch.float64)
    assert torch.allclose(f.double(), want, rtol=2e-6)
    assert f.dtype == torch.float32


def test_rope_equals_slow_form_and_is_split_half():
    # candle-nn/tests/ops.rs:185-210 compares rope with rope_slow on (2,5,10,16)-shaped data
    torch.manual_seed(299792458)
    x = torch.rand(5, 10, 16)
    cos, sin = torch.rand(10, 8), torch.rand(10, 8)
    assert torch.equal(pm.rope_half(x, cos, sin), pm.rope_slow(x, cos, sin))
    # pairing is (i, i + d/2): rotating a vector with one non-zero feature moves it there
    e = torch.zeros(1, 1, 16); e[0, 0, 3] = 1.0
    c, s = torch.zeros(1, 8), torch.ones(1, 8)
    out = pm.rope_half(e, c, s)
    assert out[0, 0, 3 + 8].item() == 1.0 and out.abs().sum().item() == 1.0
    out_i = pm.rope_interleaved(e, c, s)
    assert out_i[0, 0, 2].item() == -1.0            # the other pairing puts it elsewhere


def test_rope_position_zero_norm_and_relative_property():
    torch.manual_seed(1)
    q, k = torch.randn(1, 1, 32, dtype=torch.float64), torch.randn(1, 1, 32, dtype=torch.float64)
    def rot(x, p):
        cos, sin = pm.rope_tables(torch.tensor([p]), 10000.0, 32)
        return pm.rope_half(x, cos.double(), sin.double())
    assert torch.allclose(rot(q, 0), q)
    assert torch.allclose(rot(q, 17).norm(), q.norm())
    a = (rot(q, 40) * rot(k, 33)).sum()
    b = (rot(q, 107) * rot(k, 100)).sum()
    assert torch.allclose(a, b, atol=1e-5)           # only the distance counts
    c = (rot(q, 33) * rot(k, 40)).sum()
    assert not torch.allclose(a, c, atol=1e-3)       # and its sign


def test_attention_reduces_to_library_sdpa():
    torch.manual_seed(2)
    q, k, v = torch.randn(4, 9, 16), torch.randn(4, 9, 16), torch.randn(4, 9, 16)
    want = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    assert torch.allclose(pm.attention_core(q, k, v), want, atol=1e-5)
    nomask = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None])[0]
    assert torch.allclose(pm.attention_core(q, k, v, masked=False), nomask, atol=1e-5)
    # a portion with offset: rows see keys j <= offset + i
    off = 5
    mask = torch.arange(9)[None, :] <= (torch.arange(4)[:, None] + off)
    want = torch.nn.functional.scaled_dot_product_attention(q[None, :, :4], k[None], v[None], attn_mask=mask)[0]
    assert torch.allclose(pm.attention_core(q[:, :4], k, v, offset=off), want, atol=1e-5)
    # first token attends to itself alone
    assert torch.allclose(pm.attention_core(q, k, v)[:, 0], v[:, 0], atol=1e-6)


def test_gqa_head_mapping():
    # query head h reads kv head h // g: make kv heads distinguishable constants
    nq, nkv, t, d = 6, 3, 4, 8
    q = torch.randn(nq, t, d)
    k = torch.randn(nkv, t, d)
    v = torch.stack([torch.full((t, d), float(h + 1)) for h in range(nkv)])
    out = pm.attention_core(q, k, v)
    for h in range(nq):
        assert torch.allclose(out[h], torch.full((t, d), float(h // 2 + 1)))
    r = pm.repeat_kv(v, 2)
    assert [r[i, 0, 0].item() for i in range(6)] == [1., 1., 2., 2., 3., 3.]


def test_silu_and_mlp():
    assert pm.silu(torch.tensor(0.0)).item() == 0.0
    assert abs(pm.silu(torch.tensor(30.0)).item() - 30.0) < 1e-5
    z = torch.linspace(-6, 6, 25)
    assert torch.allclose(pm.silu(z), torch.nn.functional.silu(z), atol=1e-6)        # the library's routine
    torch.manual_seed(3)
    x = torch.randn(3, 8, dtype=torch.float64)
    g, u, d = (torch.randn(12, 8, dtype=torch.float64), torch.randn(12, 8, dtype=torch.float64),
               torch.randn(8, 12, dtype=torch.float64))
    base = pm.mlp(x, g, u, d)
    # Which of the two projections goes through the activation (attention_utils.rs:112-117: the gate): the result is
    # linear in the up projection and in the down projection, and not in the gate.  With the two swapped the first
    # line fails and the third holds.
    assert torch.allclose(pm.mlp(x, g, 3.0 * u, d), 3.0 * base, atol=1e-12)
    assert torch.allclose(pm.mlp(x, g, u, -2.0 * d), -2.0 * base, atol=1e-12)
    assert not torch.allclose(pm.mlp(x, 3.0 * g, u, d), 3.0 * base, atol=1e-3)
    # a gate that is shut (a large negative product) closes the unit whatever the up projection holds
    shut = pm.mlp(torch.ones(1, 8, dtype=torch.float64), -40.0 * torch.ones(12, 8, dtype=torch.float64), u, d)
    assert float(shut.abs().max()) < 1e-9
    # and a wide-open gate lets gate * up through: silu(z) -> z
    x1 = torch.ones(1, 8, dtype=torch.float64)
    g1 = 5.0 * torch.ones(12, 8, dtype=torch.float64)
    assert torch.allclose(pm.mlp(x1, g1, u, d), pm.linear(pm.linear(x1, g1) * pm.linear(x1, u), d), rtol=1e-12)


def _layer_parts(seed=0, nq=4, nkv=2, d=8, hidden=24, t=9, spread=0.5):
    """Random weights of one attention layer with norm weights that differ within every rotary pair."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rms_norm_eps=1e-6)
    p = {"q_proj.weight": rn(nq * d, hidden), "k_proj.weight": rn(nkv * d, hidden), "v_proj.weight": rn(nkv * d, hidden),
         "o_proj.weight": rn(hidden, nq * d), "q_norm.weight": 1.0 + spread * rn(d), "k_norm.weight": 1.0 + spread * rn(d)}
    return cfg, p, rn(t, hidden)


def _tables(positions, d):
    cos, sin = pm.rope_tables(torch.as_tensor(positions), 10000.0, d)
    return cos.double(), sin.double()


def test_attention_layer_counts_distances_only():
    """Rotary attention sees distances between positions, never positions themselves: shifting every position by
    the same amount changes nothing.  That holds when the per-head norm comes BEFORE the rotation
    (qwen3.rs:128-135).  Were the norm applied after it, its weights, which differ within a rotated pair, would
    scale the two halves of a pair differently and the scores would depend on the positions themselves: the
    variant below, with the two steps in the other order, fails the same check."""
    cfg, p, x = _layer_parts()
    d = cfg["head_dim"]
    here = pm.attention_layer(x, p, "", cfg, *_tables(range(9), d))
    there = pm.attention_layer(x, p, "", cfg, *_tables(range(1000, 1009), d))
    # (the angles are formed in 32-bit, as the reference forms them: at position 1,000 they are rounded to 6e-5)
    assert float((here - there).abs().max()) < 1e-5 * float(here.abs().max())

    def norm_after_rotation(x, cos, sin):
        t, nq, nkv = x.shape[0], cfg["num_attention_heads"], cfg["num_key_value_heads"]
        q = pm.linear(x, p["q_proj.weight"]).reshape(t, nq, d).transpose(0, 1)
        k = pm.linear(x, p["k_proj.weight"]).reshape(t, nkv, d).transpose(0, 1)
        v = pm.linear(x, p["v_proj.weight"]).reshape(t, nkv, d).transpose(0, 1)
        q = pm.rms_norm(pm.rope_half(q, cos, sin), p["q_norm.weight"], 1e-6)
        k = pm.rms_norm(pm.rope_half(k, cos, sin), p["k_norm.weight"], 1e-6)
        return pm.linear(pm.attention_core(q, k, v).transpose(0, 1).reshape(t, nq * d), p["o_proj.weight"])
    wrong_here = norm_after_rotation(x, *_tables(range(9), d))
    wrong_there = norm_after_rotation(x, *_tables(range(1000, 1009), d))
    assert float((wrong_here - wrong_there).abs().max()) > 1e-2 * float(wrong_here.abs().max())
    assert float((wrong_here - here).abs().max()) > 1e-2 * float(here.abs().max())


def test_attention_layer_norms_queries_and_keys_per_head_and_not_values():
    """What the per-head norm covers (qwen3.rs:128-129, attention_utils.rs:52-58): queries and keys, each head on
    its own, values not.  So the layer does not notice a rescaled query or key head (a norm over all heads
    together would, and so would no norm), and it is linear in the value projection (a normed value would not be)."""
    cfg, p, x = _layer_parts(seed=1)
    cfg["rms_norm_eps"] = 1e-14                                 # (so that a head's scale drops out exactly)
    d = cfg["head_dim"]
    tables = _tables(range(9), d)
    base = pm.attention_layer(x, p, "", cfg, *tables)
    scaled = dict(p)
    scaled["q_proj.weight"] = p["q_proj.weight"].clone()
    scaled["q_proj.weight"][d:2 * d] *= 7.0                     # query head 1 alone
    scaled["k_proj.weight"] = p["k_proj.weight"].clone()
    scaled["k_proj.weight"][:d] *= 0.2                          # key head 0 alone
    assert torch.allclose(pm.attention_layer(x, scaled, "", cfg, *tables), base, atol=1e-6)
    wide = dict(p, **{"v_proj.weight": 3.0 * p["v_proj.weight"]})
    assert torch.allclose(pm.attention_layer(x, wide, "", cfg, *tables), 3.0 * base, atol=1e-9)
    # one weight vector of head_dim entries serves every head
    assert p["q_norm.weight"].shape == (d,)
    # and it matters: other norm weights, other result
    other = dict(p, **{"q_norm.weight": p["q_norm.weight"].flip(0)})
    assert float((pm.attention_layer(x, other, "", cfg, *tables) - base).abs().max()) > 1e-3 * float(base.abs().max())


def test_decoder_layer_keeps_the_stream_beside_its_parts():
    """Pre-norm residuals (qwen3.rs:284-300): the stream goes round both parts untouched, and the norms stand on the
    parts' inputs.  With output projections of zero the layer is the identity (a norm on the stream itself, or after
    the sum, would change x); and what a part adds is a function of the NORMED stream: scaling the stream by a
    constant scales the layer's additions not at all."""
    torch.manual_seed(5)
    cfg = dict(num_attention_heads=4, num_key_value_heads=2, head_dim=8, rms_norm_eps=1e-9, hidden_size=24)
    rn = lambda *s: torch.randn(*s, dtype=torch.float64)
    pre = "model.layers.0."
    p = {pre + "self_attn.q_proj.weight": rn(32, 24), pre + "self_attn.k_proj.weight": rn(16, 24),
         pre + "self_attn.v_proj.weight": rn(16, 24), pre + "self_attn.o_proj.weight": rn(24, 32),
         pre + "self_attn.q_norm.weight": 1 + 0.3 * rn(8), pre + "self_attn.k_norm.weight": 1 + 0.3 * rn(8),
         pre + "input_layernorm.weight": 1 + 0.3 * rn(24), pre + "post_attention_layernorm.weight": 1 + 0.3 * rn(24),
         pre + "mlp.gate_proj.weight": rn(40, 24), pre + "mlp.up_proj.weight": rn(40, 24),
         pre + "mlp.down_proj.weight": rn(24, 40)}
    x = rn(7, 24)
    tables = _tables(range(7), 8)
    silent = dict(p)
    silent[pre + "self_attn.o_proj.weight"] = torch.zeros(24, 32, dtype=torch.float64)
    silent[pre + "mlp.down_proj.weight"] = torch.zeros(24, 40, dtype=torch.float64)
    assert torch.equal(pm.decoder_layer(x, silent, 0, cfg, *tables), x)
    # the attention part alone (the feed-forward silent): its addition does not change when the stream is scaled
    quiet_ffn = dict(p)
    quiet_ffn[pre + "mlp.down_proj.weight"] = torch.zeros(24, 40, dtype=torch.float64)
    add1 = pm.decoder_layer(x, quiet_ffn, 0, cfg, *tables) - x
    add5 = pm.decoder_layer(5.0 * x, quiet_ffn, 0, cfg, *tables) - 5.0 * x
    assert torch.allclose(add1, add5, atol=1e-7)
    # the feed-forward reads the stream AFTER the attention's addition: with the attention silent it sees norm(x),
    # with it speaking something else
    quiet_attn = dict(p)
    quiet_attn[pre + "self_attn.o_proj.weight"] = torch.zeros(24, 32, dtype=torch.float64)
    ffn_alone = pm.decoder_layer(x, quiet_attn, 0, cfg, *tables) - x
    want = pm.mlp(pm.rms_norm(x, p[pre + "post_attention_layernorm.weight"], 1e-9), p[pre + "mlp.gate_proj.weight"],
                  p[pre + "mlp.up_proj.weight"], p[pre + "mlp.down_proj.weight"])
    assert torch.allclose(ffn_alone, want, atol=1e-9)
    both = pm.decoder_layer(x, p, 0, cfg, *tables)
    mid = x + add1
    want_both = mid + pm.mlp(pm.rms_norm(mid, p[pre + "post_attention_layernorm.weight"], 1e-9),
                             p[pre + "mlp.gate_proj.weight"], p[pre + "mlp.up_proj.weight"], p[pre + "mlp.down_proj.weight"])
    assert torch.allclose(both, want_both, atol=1e-9)


def test_rand_f32_matches_integer_transcription():
    # a second, independent transcription of inferrs/src/sampler.rs:370-397 with numpy uint64
    import numpy as np
    def ref(seed, step):
        with np.errstate(over="ignore"):
            x = np.uint64(seed) + np.uint64(0x9e3779b97f4a7c15)
            for rnd in range(2):
                if rnd == 1:
                    x = x + (np.uint64(step) + np.uint64(1)) * np.uint64(0x9e3779b97f4a7c15)
                x = (x ^ (x >> np.uint64(30))) * np.uint64(0xbf58476d1ce4e5b9)
                x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94d049bb133111eb)
                x = x ^ (x >> np.uint64(31))
            x ^= x << np.uint64(13); x ^= x >> np.uint64(7); x ^= x << np.uint64(17)
            u = (x * np.uint64(0x2545f4914f6cdd1d)) >> np.uint64(32)
        return float(np.float32(u) / np.float32(4294967296.0))
    vals = [pm.rand_f32(42, s) for s in range(50)]
    assert vals == [ref(42, s) for s in range(50)]
    assert all(0.0 <= v < 1.0 for v in vals) and len(set(vals)) == 50


def test_sampler_penalty_window_and_greedy():
    # inferrs/src/sampler.rs:613-644: the window holds the last repeat_last_n tokens only
    logits = torch.zeros(8); logits[1] = 10.0; logits[2] = 9.99
    assert pm.sample(logits, [1] + [5] * 3, temperature=0.0, repetition_penalty=2.0, repeat_last_n=4) == 2
    assert pm.sample(logits, [1] + [5] * 4, temperature=0.0, repetition_penalty=2.0, repeat_last_n=4) == 1
    assert pm.sample(logits, [1], temperature=0.0, repetition_penalty=2.0, repeat_last_n=0) == 1
    tie = torch.tensor([1.0, 3.0, 3.0, 0.0])
    assert pm.sample(tie, [], temperature=0.0) == 1                  # lowest index among maxima
    assert pm.sample(torch.tensor([0.0, 50.0, 0.0]), [], temperature=1.0, top_k=1, seed=3) == 1


def test_sampler_frequencies_follow_tempered_softmax():
    logits = torch.tensor([0.0, 1.0, 2.0, -1.0])
    temp = 0.7
    want = torch.softmax(logits / temp, 0)
    counts = torch.zeros(4)
    n = 4000
    for step in range(n):
        prev = [0] * step if step < 64 else [0] * 64
        # step enters through len(previous): feed a list of that length without penalties
        t = pm.sample(logits, list(range(step % 97)), temperature=temp, top_k=0, top_p=1.0,
                      repetition_penalty=1.0, seed=step)
        counts[t] += 1
    assert torch.allclose(counts / n, want, atol=0.03)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_model_shift_and_prefix_invariants(tmp_path, name):
    raw = TINY[name]
    folder = write_model(str(tmp_path / name), raw, seed=5)
    cfg, p = pm.read_model(folder, torch.float64)
    toks = random_tokens(24, raw["vocab_size"], 7)
    full = pm.forward(cfg, p, toks)
    assert full.shape == (24, raw["vocab_size"])
    # causality: logits of a prefix do not depend on what follows
    assert torch.allclose(pm.forward(cfg, p, toks[:11]), full[:11], atol=1e-9)
    # the head: tied models use the embedding table
    if raw["tie_word_embeddings"]:
        assert "lm_head.weight" not in p
    else:
        assert p["lm_head.weight"].shape == (raw["vocab_size"], raw["hidden_size"])
    # greedy continuation feeds its own tokens back: the arg max of the logits after each of them
    out = pm.greedy(cfg, p, toks[:5], 3)
    assert out[0] == int(torch.argmax(full[4]))            # (causality: position 4 does not see what follows it)
    assert out[1] == int(torch.argmax(pm.forward(cfg, p, toks[:5] + out[:1])[-1]))
    assert out[2] == int(torch.argmax(pm.forward(cfg, p, toks[:5] + out[:2])[-1]))


def _two_ends_model(tmp_path, **changes):
    """Tiny configuration B (its head is a matrix of its own) in 64-bit, with `changes` to its config."""
    folder = write_model(str(tmp_path / "ends"), TINY["B"], seed=6)
    cfg, p = pm.read_model(folder, torch.float64)
    assert "lm_head.weight" in p and not TINY["B"]["tie_word_embeddings"]
    return dict(cfg, **changes), p


def test_final_norm_stands_before_the_head(tmp_path):
    """`x = norm(x)` before the logits (qwen3.rs:398-405, attention_utils.rs:382-395).  Scale the embedding table and
    every output projection (o_proj, down_proj) by c: every part reads the normed stream, so each addition and the
    stream itself become c times what they were, and a norm in front of the head takes the factor out again: the
    logits do not change.  Without the final norm they would be c times as large; with a norm applied to something
    else than the final stream (only the last layer's addition, say) the factor would survive as well."""
    cfg, p = _two_ends_model(tmp_path, rms_norm_eps=1e-14)            # (so that a scale drops out exactly)
    toks = random_tokens(19, TINY["B"]["vocab_size"], 3)
    base = pm.forward(cfg, p, toks)
    c = 7.0
    scaled = {k: (c * v if k == "model.embed_tokens.weight" or k.endswith(("o_proj.weight", "down_proj.weight")) else v)
              for k, v in p.items()}
    assert float((pm.forward(cfg, scaled, toks) - base).abs().max()) < 1e-9 * float(base.abs().max())
    # the check can fail: scale the head instead and the logits follow
    louder = dict(p, **{"lm_head.weight": c * p["lm_head.weight"]})
    assert torch.allclose(pm.forward(cfg, louder, toks), c * base, rtol=1e-12)


def test_embedding_enters_the_stream_unscaled(tmp_path):
    """`x = embed(ids)` and nothing else (qwen3.rs:398-400: no sqrt(hidden) factor as other families have).  With
    output projections of zero the stream is the embedding row itself, and with an eps so large that the norm's
    divisor is sqrt(eps) the logits are (E[id] * w_final) . W_head^T / sqrt(eps) in plain arithmetic: a factor on the
    embedding would show one to one."""
    eps = 1e6
    cfg, p = _two_ends_model(tmp_path, rms_norm_eps=eps)
    silent = {k: (torch.zeros_like(v) if k.endswith(("o_proj.weight", "down_proj.weight")) else v) for k, v in p.items()}
    toks = random_tokens(13, TINY["B"]["vocab_size"], 4)
    got = pm.forward(cfg, silent, toks)
    rows = p["model.embed_tokens.weight"][torch.as_tensor(toks)]
    want = (rows * p["model.norm.weight"]) @ p["lm_head.weight"].T / eps ** 0.5
    assert float((got - want).abs().max()) < 1e-6 * float(want.abs().max())
    hidden = TINY["B"]["hidden_size"]
    assert float((got - want * hidden ** 0.5).abs().max()) > 0.5 * float(want.abs().max())     # what a scaled embedding would give
