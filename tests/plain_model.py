"""A plain, slow implementation of the Qwen3 dense decoder, written from the reference's formulas.

Whole sequences, no cache, no paging, one function per part, plain torch tensor arithmetic on
the CPU.  It shares no code with `inferrs_amd`: the model folder is read with the `safetensors`
package and `json`, the configuration keys are taken straight from config.json.  Every function
cites the lines of the reference it transcribes (paths relative to the reference's root).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# ---- parts ----------------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * w over the last dimension.
    candle-nn/src/ops.rs:480-490 (CPU), inferrs-kernels/candle-kernels/src/reduce.cu:189-228."""
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(mean_sq + eps) * w


def inv_freq(theta: float, rot_dim: int) -> torch.Tensor:
    """1 / theta^(2i/rot_dim), i in [0, rot_dim/2), every operation on float32 values with a
    correctly rounded powf (the power is taken in float64 and rounded once).
    inferrs-models/src/models/attention_utils.rs:198-203."""
    out = []
    base = torch.tensor(theta, dtype=torch.float32).double()
    for i in range(rot_dim // 2):
        exp = torch.tensor(2.0 * i, dtype=torch.float32) / torch.tensor(float(rot_dim), dtype=torch.float32)
        out.append(torch.tensor(1.0, dtype=torch.float32) / torch.pow(base, exp.double()).float())
    return torch.stack(out)


def rope_tables(positions: torch.Tensor, theta: float, rot_dim: int):
    """cos/sin of position * inv_freq, float32.  attention_utils.rs:205-215."""
    ang = positions.to(torch.float32).unsqueeze(1) * inv_freq(theta, rot_dim).unsqueeze(0)
    return torch.cos(ang), torch.sin(ang)


def rope_half(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Split-half rotation of x [heads, t, d] with cos/sin [t, d/2]:
    out[i] = x[i]c - x[i+d/2]s, out[i+d/2] = x[i]s + x[i+d/2]c.
    inferrs-kernels/candle-kernels/src/reduce.cu:292-312; attention_utils.rs:137-181."""
    d = x.shape[-1]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    c, s = cos.to(x.dtype), sin.to(x.dtype)
    return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1)


def rope_slow(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """The reference's check form x*[cos,cos] + rotate_half(x)*[sin,sin], rotate_half = [-x2, x1].
    candle-nn/src/rotary_emb.rs:540-556."""
    d = x.shape[-1]
    c = torch.cat([cos, cos], dim=-1).to(x.dtype)
    s = torch.cat([sin, sin], dim=-1).to(x.dtype)
    rot = torch.cat([-x[..., d // 2:], x[..., : d // 2]], dim=-1)
    return x * c + rot * s


def rope_interleaved(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Pairs (2i, 2i+1): reduce.cu:275-289.  Not used by Qwen3; here to tell the pairings apart."""
    x1, x2 = x[..., 0::2], x[..., 1::2]
    c, s = cos.to(x.dtype), sin.to(x.dtype)
    return torch.stack([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1).flatten(-2)


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[kv, t, d] -> [kv*n_rep, t, d], each kv head repeated consecutively, so query head h
    reads kv head h // n_rep.  attention_utils.rs:38-49."""
    kv, t, d = x.shape
    return x.unsqueeze(1).expand(kv, n_rep, t, d).reshape(kv * n_rep, t, d)


def causal_mask(q_len: int, kv_len: int, offset: int, dtype=torch.float32) -> torch.Tensor:
    """0 where j <= offset + i, -inf elsewhere.  attention_utils.rs:61-85."""
    i = torch.arange(q_len).unsqueeze(1) + offset
    j = torch.arange(kv_len).unsqueeze(0)
    return torch.where(j <= i, torch.zeros((), dtype=dtype), torch.full((), float("-inf"), dtype=dtype))


def softmax_last(x: torch.Tensor) -> torch.Tensor:
    """exp(x - max) / sum.  candle-nn/src/ops.rs:283-313, reduce.cu:233-272."""
    m = x.max(dim=-1, keepdim=True).values
    e = torch.exp(x - m)
    return e / e.sum(dim=-1, keepdim=True)


def attention_core(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, offset: int = 0,
                   scale: Optional[float] = None, masked: bool = True) -> torch.Tensor:
    """q [nq, t, d], k/v [nkv, kv, d] -> [nq, t, d].  Scores are scaled after the product by
    1/sqrt(d); the mask is added when t > 1.  inferrs-models/src/models/qwen3.rs:163-186."""
    nq, t, d = q.shape
    g = nq // k.shape[0]
    k, v = repeat_kv(k, g), repeat_kv(v, g)
    s = torch.matmul(q, k.transpose(1, 2)) * (1.0 / math.sqrt(d) if scale is None else scale)
    if masked and t > 1:
        s = s + causal_mask(t, k.shape[1], offset, s.dtype)
    return torch.matmul(softmax_last(s), v)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x . W^T with W [out, in].  candle-nn/src/linear.rs:64-72."""
    return torch.matmul(x, w.t())


def silu(z: torch.Tensor) -> torch.Tensor:
    """z / (1 + exp(-z)).  inferrs-kernels/candle-kernels/src/unary.cu:59-61."""
    return z / (1.0 + torch.exp(-z))


def mlp(x: torch.Tensor, gate_w, up_w, down_w) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)).  attention_utils.rs:112-117."""
    return linear(silu(linear(x, gate_w)) * linear(x, up_w), down_w)


def attention_layer(x: torch.Tensor, p: Dict[str, torch.Tensor], prefix: str, cfg: Dict,
                    cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Projections, per-head q/k norm, rotation, attention, output projection for a whole
    sequence x [t, hidden].  qwen3.rs:105-195."""
    t = x.shape[0]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = linear(x, p[prefix + "q_proj.weight"]).reshape(t, nq, d).transpose(0, 1)
    k = linear(x, p[prefix + "k_proj.weight"]).reshape(t, nkv, d).transpose(0, 1)
    v = linear(x, p[prefix + "v_proj.weight"]).reshape(t, nkv, d).transpose(0, 1)
    q = rms_norm(q, p[prefix + "q_norm.weight"], cfg["rms_norm_eps"])      # qwen3.rs:128
    k = rms_norm(k, p[prefix + "k_norm.weight"], cfg["rms_norm_eps"])      # qwen3.rs:129
    q, k = rope_half(q, cos, sin), rope_half(k, cos, sin)                  # qwen3.rs:132-135
    o = attention_core(q, k, v, offset=0)
    o = o.transpose(0, 1).reshape(t, nq * d)                               # qwen3.rs:189-192
    return linear(o, p[prefix + "o_proj.weight"])


def decoder_layer(x: torch.Tensor, p: Dict[str, torch.Tensor], i: int, cfg: Dict, cos, sin) -> torch.Tensor:
    """x + attn(norm(x)); then x + mlp(norm(x)).  qwen3.rs:284-300."""
    pre = f"model.layers.{i}."
    h = rms_norm(x, p[pre + "input_layernorm.weight"], cfg["rms_norm_eps"])
    x = x + attention_layer(h, p, pre + "self_attn.", cfg, cos, sin)
    h = rms_norm(x, p[pre + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    return x + mlp(h, p[pre + "mlp.gate_proj.weight"], p[pre + "mlp.up_proj.weight"],
                   p[pre + "mlp.down_proj.weight"])


# ---- the whole model --------------------------------------------------------------------------

def read_model(model_dir: str, dtype=torch.float32):
    """config.json as a dict with the reference's defaults filled in
    (inferrs-models/src/config.rs:468-502), and the tensors widened to `dtype`."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])
    if cfg.get("head_dim") is None:
        cfg["head_dim"] = cfg["hidden_size"] // cfg["num_attention_heads"]
    cfg.setdefault("rms_norm_eps", 1e-6)
    cfg.setdefault("rope_theta", 1_000_000.0)
    tensors = {k: v.to(dtype) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, tensors


def forward(cfg: Dict, p: Dict[str, torch.Tensor], token_ids: Sequence[int]) -> torch.Tensor:
    """Logits [t, vocab] at every position of one whole sequence.  qwen3.rs:398-407; the
    logits head falls back to the embedding table when lm_head.weight is absent
    (qwen3.rs:369-372).  The reference returns the last row only (attention_utils.rs:382-395)."""
    ids = torch.as_tensor(list(token_ids), dtype=torch.long)
    dtype = p["model.embed_tokens.weight"].dtype
    x = p["model.embed_tokens.weight"][ids]
    cos, sin = rope_tables(torch.arange(len(ids)), float(cfg["rope_theta"]), cfg["head_dim"])
    cos, sin = cos.to(dtype), sin.to(dtype)
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, p, i, cfg, cos, sin)
    x = rms_norm(x, p["model.norm.weight"], cfg["rms_norm_eps"])
    head = p.get("lm_head.weight", p["model.embed_tokens.weight"])
    return linear(x, head)


def greedy(cfg: Dict, p: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int) -> List[int]:
    """Greedy continuation by re-running the whole sequence; lowest index among equal maxima
    (candle-core/src/cpu_backend/mod.rs:150-157)."""
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(cfg, p, toks)[-1])))
    return toks[len(prompt):]


# ---- sampling ---------------------------------------------------------------------------------

_M64 = (1 << 64) - 1


def rand_f32(seed: int, step: int) -> float:
    """inferrs/src/sampler.rs:370-397 for a given seed."""
    def mix(x):
        x = ((x ^ (x >> 30)) * 0xbf58476d1ce4e5b9) & _M64
        x = ((x ^ (x >> 27)) * 0x94d049bb133111eb) & _M64
        return x ^ (x >> 31)
    x = mix((seed + 0x9e3779b97f4a7c15) & _M64)
    x = mix((x + ((step + 1) * 0x9e3779b97f4a7c15 & _M64)) & _M64)
    if x == 0:
        x = 0x1234567890abcdef
    x ^= (x << 13) & _M64
    x ^= x >> 7
    x ^= (x << 17) & _M64
    u = ((x * 0x2545f4914f6cdd1d) & _M64) >> 32
    return float(torch.tensor(u, dtype=torch.float64).to(torch.float32) / torch.tensor(4294967296.0))


def sample(logits: torch.Tensor, previous: Sequence[int], *, temperature=0.7, top_p=0.9, top_k=50,
           min_p=0.0, repetition_penalty=1.1, repeat_last_n=64, frequency_penalty=0.0,
           presence_penalty=0.0, seed: int = 0, logprobs: bool = False, top_logprobs: int = 0, logit_bias=None):
    """inferrs/src/sampler.rs:146-352, step by step, for a seeded request.  With `logprobs` the result is
    (token, its log-probability, [(id, log-probability)] of the kept list's first entries)."""
    z = logits.to(torch.float32).clone()
    vocab = z.numel()
    window = list(previous[-repeat_last_n:]) if repeat_last_n > 0 else []
    has_pen = (repetition_penalty != 1.0 or frequency_penalty != 0.0 or presence_penalty != 0.0) and window
    if temperature < 1e-5 and not has_pen and not logit_bias and not logprobs:      # :175-179
        return int(torch.argmax(z))
    for t, b in (logit_bias or {}).items():                                 # :185-190
        if t < vocab:
            z[t] = z[t] + torch.tensor(b, dtype=torch.float32)
    if repetition_penalty not in (1.0, 0.0) and window:                    # :196-209
        for t in dict.fromkeys(window):
            if t < vocab:
                z[t] = z[t] / repetition_penalty if z[t] >= 0 else z[t] * repetition_penalty
    if (frequency_penalty != 0.0 or presence_penalty != 0.0) and window:    # :213-229
        for t in set(window):
            if t < vocab:
                z[t] = z[t] - torch.tensor(frequency_penalty, dtype=torch.float32) * window.count(t)
                z[t] = z[t] - torch.tensor(presence_penalty, dtype=torch.float32)
    z = z / torch.tensor(max(temperature, 1e-5), dtype=torch.float32)       # :232-239
    probs = torch.exp(z - z.max())
    probs = probs / probs.sum()                                             # :242-249
    order = sorted(range(vocab), key=lambda i: -float(probs[i]))            # stable: :252-253
    kept = [(i, probs[i].item()) for i in order]
    if 0 < top_k < len(kept):
        kept = kept[:top_k]                                                 # :256-258
    if top_p < 1.0:                                                         # :261-272
        cum, cut = torch.tensor(0.0), len(kept)
        for n, (_, pr) in enumerate(kept):
            cum = cum + torch.tensor(pr, dtype=torch.float32)
            if cum >= torch.tensor(top_p, dtype=torch.float32):
                cut = n + 1
                break
        kept = kept[:cut]
    if min_p > 0.0 and kept:                                                # :277-283
        thr = torch.tensor(kept[0][1], dtype=torch.float32) * torch.tensor(min_p, dtype=torch.float32)
        cut = sum(1 for _, pr in kept if torch.tensor(pr, dtype=torch.float32) >= thr)
        if cut > 0:
            kept = kept[:cut]
    total = torch.tensor(0.0)
    for _, pr in kept:
        total = total + torch.tensor(pr, dtype=torch.float32)
    denom = float(total) if total > 0 else 1.0                             # :286-292
    top = [(i, math.log(pr / denom) if pr > 0 else -math.inf) for i, pr in kept[:top_logprobs]] if logprobs else []
    if total <= 0:
        first = kept[0][0] if kept else 0
        return (first, -math.inf, top) if logprobs else first
    u = torch.tensor(rand_f32(seed, len(previous)), dtype=torch.float32)    # :323-335
    chosen = kept[-1][0]
    for i, pr in kept:
        norm = torch.tensor(pr, dtype=torch.float32) / total
        if u < norm:
            chosen = i
            break
        u = u - norm
    if not logprobs:
        return chosen
    pr = dict(kept)[chosen] / float(total)                                  # :339-352
    return chosen, (math.log(pr) if pr > 0 else -math.inf), top
