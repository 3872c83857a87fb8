"""Each part of a layer alone against its plain formula, and the generality of the assembly:
a toy mixer with state of its own, a layer that reads another layer's cache, and a layer that
runs twice, registered and built from a test without a change to the framework's files."""
import io
import os
from dataclasses import dataclass
from typing import Any, Dict, Tuple

import numpy as np
import pytest
import torch

import plain_model as pm
import trace_modes as tm
from tiny_configs import TINY_B, random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def rel_err(got, want):
    got, want = got.detach().float().cpu().double(), want.double()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-9))


TOL = {torch.float32: 2e-6, torch.bfloat16: 2 ** -7}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from inferrs_amd.config import NormSpec
    from inferrs_amd.parts import part_class
    spec = NormSpec(size=96, eps=1e-5)
    w = rnd(96, seed=1) * 0.1 + 1
    norm = part_class("norm", spec)(spec, {"weight": w.to(torch.bfloat16)}, dtype, DEV)
    x, d = rnd(9, 96, seed=2, dtype=dtype), rnd(9, 96, seed=3, dtype=dtype)
    wq = w.to(torch.bfloat16).double()
    assert rel_err(norm.forward(x.to(DEV)), pm.rms_norm(x.double(), wq, 1e-5)) < TOL[dtype]
    xs = x.to(DEV)
    out = norm.add_forward(xs, d.to(DEV))
    summed = (x.float() + d.float()).to(dtype)
    assert torch.equal(xs.cpu(), summed)
    assert rel_err(out, pm.rms_norm(summed.double(), wq, 1e-5)) < TOL[dtype]
    # the other convention of storing the weight (w - 1) is a parameter of the part, not another part
    plus = part_class("norm", spec)(NormSpec(size=96, eps=1e-5, add_one=True), {"weight": w - 1}, dtype, DEV)
    assert rel_err(plus.forward(x.to(DEV)), pm.rms_norm(x.double(), w.double(), 1e-5)) < 2 * TOL[dtype]


def test_position_part():
    from inferrs_amd.config import PositionSpec
    from inferrs_amd.parts import part_class
    spec = PositionSpec(kind="rope", head_dim=32, rot_dim=32, theta=1e6)
    rope = part_class("position", spec)(spec, {}, torch.float32, DEV)
    assert torch.equal(rope.inv_freq.cpu(), pm.inv_freq(1e6, 32))
    pos = torch.tensor([0, 3, 999, 12345], dtype=torch.int32)
    cos, sin = rope.table(pos.to(DEV))
    want_cos, want_sin = pm.rope_tables(pos, 1e6, 32)
    assert float((cos.cpu() - want_cos).abs().max()) < 2e-6 and float((sin.cpu() - want_sin).abs().max()) < 2e-6
    none = part_class("position", PositionSpec(kind="none"))(PositionSpec(kind="none"), {}, torch.float32, DEV)
    assert none.table(pos.to(DEV)) is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    from inferrs_amd.config import GatedMlpSpec
    from inferrs_amd.parts import part_class
    spec = GatedMlpSpec(hidden=72, intermediate=200)
    t = {"gate_proj.weight": rnd(200, 72, seed=1, scale=0.1, dtype=torch.bfloat16),
         "up_proj.weight": rnd(200, 72, seed=2, scale=0.1, dtype=torch.bfloat16),
         "down_proj.weight": rnd(72, 200, seed=3, scale=0.1, dtype=torch.bfloat16)}
    ffn = part_class("ffn", spec)(spec, dict(t), dtype, DEV)
    x = rnd(11, 72, seed=4, dtype=dtype)
    want = pm.mlp(x.double(), t["gate_proj.weight"].double(), t["up_proj.weight"].double(), t["down_proj.weight"].double())
    assert rel_err(ffn.forward(None, x.to(DEV)), want) < 2 * TOL[dtype]


def attention_setup(dtype, page_size, spec, tensors, requests):
    """A cache of its own for one attention part, and the step contexts to run `requests`
    (name -> (tokens' hidden rows, cut points)) through it."""
    from inferrs_amd.cache import CacheManager, CacheStorage
    from inferrs_amd.engine import StepBuilder
    from inferrs_amd.parts import part_class
    cls = part_class("mixer", spec)
    manager = CacheManager({0: cls.cache_need(spec)}, page_size, 64, 4)
    storage = CacheStorage(manager, dtype, DEV)
    return cls(spec, dict(tensors), dtype, DEV), manager, storage, StepBuilder(manager, DEV)


@pytest.mark.parametrize("dtype,page", [(torch.float32, 4), (torch.bfloat16, 16), (torch.bfloat16, 8)])
def test_attention_part(dtype, page):
    """The mixer alone, over its own cache, in two steps (a portion, then the rest beside a
    second request), against the plain attention layer on the whole sequences."""
    from inferrs_amd.config import AttentionSpec, NormSpec, PositionSpec
    cfg = dict(num_attention_heads=6, num_key_value_heads=3, head_dim=32, rms_norm_eps=1e-5)
    hidden = 96
    spec = AttentionSpec(hidden=hidden, n_heads=6, n_kv_heads=3, head_dim=32,
                         position=PositionSpec(kind="rope", head_dim=32, rot_dim=32, theta=1e4),
                         qk_norm=NormSpec(size=32, eps=1e-5))
    t = {"q_proj.weight": rnd(192, hidden, seed=1, scale=0.1, dtype=torch.bfloat16),
         "k_proj.weight": rnd(96, hidden, seed=2, scale=0.1, dtype=torch.bfloat16),
         "v_proj.weight": rnd(96, hidden, seed=3, scale=0.1, dtype=torch.bfloat16),
         "o_proj.weight": rnd(hidden, 192, seed=4, scale=0.1, dtype=torch.bfloat16),
         "q_norm.weight": (rnd(32, seed=5) * 0.1 + 1).to(torch.bfloat16),
         "k_norm.weight": (rnd(32, seed=6) * 0.1 + 1).to(torch.bfloat16)}
    attn, manager, storage, builder = attention_setup(dtype, page, spec, t, None)
    ha, hb = rnd(37, hidden, seed=7, dtype=dtype), rnd(5, hidden, seed=8, dtype=dtype)
    outs = {"a": [], "b": []}
    for step in ([("a", ha[:20])], [("a", ha[20:]), ("b", hb)]):
        for name, rows in step:
            if name not in manager.sequences:
                manager.add_sequence(name)
            assert manager.reserve(name, rows.shape[0])
        ctx = builder.build([(name, [0] * rows.shape[0], []) for name, rows in step])
        y = attn.forward(ctx, torch.cat([rows for _, rows in step]).to(DEV), storage.layers[0])
        off = 0
        for name, rows in step:
            outs[name].append(y[off:off + rows.shape[0]].cpu())
            off += rows.shape[0]
            manager.commit(name, rows.shape[0])
    p = {"x." + k: v.double() for k, v in t.items()}
    for name, h in (("a", ha), ("b", hb)):
        cos, sin = pm.rope_tables(torch.arange(h.shape[0]), 1e4, 32)
        want = pm.attention_layer(h.double(), p, "x.", cfg, cos.double(), sin.double())
        assert rel_err(torch.cat(outs[name]), want) < 4 * TOL[dtype], name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_part_without_norm_or_rotation_is_plain_attention(dtype):
    """With no per-head norm and no position encoding the mixer reduces to a library routine."""
    from inferrs_amd.config import AttentionSpec, PositionSpec
    hidden, nq, nkv, d = 64, 4, 4, 16
    spec = AttentionSpec(hidden=hidden, n_heads=nq, n_kv_heads=nkv, head_dim=d, position=PositionSpec(kind="none"))
    eye = torch.eye(hidden, dtype=torch.bfloat16)
    t = {"q_proj.weight": eye, "k_proj.weight": eye, "v_proj.weight": eye, "o_proj.weight": eye}
    attn, manager, storage, builder = attention_setup(dtype, 16, spec, t, None)
    h = rnd(50, hidden, seed=9, dtype=dtype)
    manager.add_sequence("a")
    manager.reserve("a", 50)
    y = attn.forward(builder.build([("a", [0] * 50, [])]), h.to(DEV), storage.layers[0])
    q = h.double().view(50, nq, d).transpose(0, 1)
    want = torch.nn.functional.scaled_dot_product_attention(q, q, q, is_causal=True).transpose(0, 1).reshape(50, hidden)
    assert rel_err(y, want) < 4 * TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_alone(dtype, tmp_path):
    """One block built from a layer spec equals the plain decoder layer."""
    from inferrs_amd.cache import CacheManager, CacheStorage
    from inferrs_amd.config import Qwen3Config
    from inferrs_amd.engine import StepBuilder
    from inferrs_amd.parts import Block, layer_tensors, part_class
    from inferrs_amd.weights import random_tensors
    cfg = Qwen3Config.from_dict(TINY_B)
    layer = cfg.to_spec().layers[1]
    tensors = random_tensors(layer_tensors(layer), 3, torch.bfloat16)
    block = Block(layer, dict(tensors), dtype, DEV)
    manager = CacheManager({0: part_class("mixer", layer.mixer).cache_need(layer.mixer)}, 16, 8, 2)
    storage = CacheStorage(manager, dtype, DEV)
    x = rnd(23, cfg.hidden_size, seed=5, dtype=dtype)
    manager.add_sequence("a")
    manager.reserve("a", 23)
    ctx = StepBuilder(manager, DEV).build([("a", [0] * 23, [])])
    stream, pending = block.forward(ctx, x.to(DEV).clone(), None, storage.layers[0])
    cos, sin = pm.rope_tables(torch.arange(23), cfg.rope_theta, cfg.head_dim)
    want = pm.decoder_layer(x.double(), {k: v.double() for k, v in tensors.items()}, 1, TINY_B, cos.double(), sin.double())
    assert rel_err(stream.float() + pending.float(), want) < 4 * TOL[dtype]


# ---- a toy architecture, defined here ---------------------------------------------------------

@dataclass(frozen=True)
class CumMeanSpec:
    """A mixer with state of its own: out[t] = W . mean(h[0..t]).  It keeps the running sum and
    the count per request, not keys and values."""
    hidden: int
    kind: str = "toy_cummean"


def register_toy():
    from inferrs_amd import ops
    from inferrs_amd.config import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                                    ScheduleEntry)
    from inferrs_amd.config.registry import register_architecture
    from inferrs_amd.parts import FixedState, Mixer, register_mixer
    from inferrs_amd.weights import TensorSpec

    @register_mixer("toy_cummean")
    class CumMean(Mixer):
        @classmethod
        def tensors(cls, spec):
            return {"mix.weight": TensorSpec((spec.hidden, spec.hidden))}

        @classmethod
        def cache_need(cls, spec):
            return FixedState((spec.hidden + 1,), torch.float32)

        def __init__(self, spec, tensors, dtype, device):
            self.spec = spec
            self.w = tensors["mix.weight"].to(device=device, dtype=dtype).contiguous()

        def forward(self, ctx, h, cache):
            out = torch.empty_like(h)
            off = 0
            for n, slot in zip(ctx.q_lens, ctx.state_slots_host):      # a toy: one request at a time
                state = cache.state[slot]
                sums = state[:-1] + torch.cumsum(h[off:off + n].float(), 0)
                counts = state[-1] + torch.arange(1, n + 1, device=h.device, dtype=torch.float32)
                out[off:off + n] = (sums / counts[:, None]).to(h.dtype)
                state[:-1] = sums[-1]
                state[-1] = counts[-1]
                off += n
            return ops.linear(out, self.w)

    class ToyConfig:
        architecture = "ToyForCausalLM"
        model_type = "toy"

        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def to_dict(self):
            return dict(self.raw, architectures=[self.architecture], model_type=self.model_type)

        def to_spec(self):
            r = self.raw
            h = r["hidden_size"]
            norm = NormSpec(size=h, eps=r["eps"])
            attn = AttentionSpec(hidden=h, n_heads=r["heads"], n_kv_heads=r["kv_heads"], head_dim=r["head_dim"],
                                 position=PositionSpec(kind="rope", head_dim=r["head_dim"], rot_dim=r["head_dim"] // 2,
                                                       theta=100.0),
                                 qk_norm=None, window=r["window"])
            ffn = GatedMlpSpec(hidden=h, intermediate=r["intermediate"])

            def layer(i, mixer):
                p = f"blocks.{i}."
                return LayerSpec(mixer=mixer, ffn=ffn, norms=(norm, norm), norm_names=(p + "norm1.weight", p + "norm2.weight"),
                                 mixer_prefix=p + "mixer.", ffn_prefix=p + "ffn.")
            layers = (layer(0, attn), layer(1, CumMeanSpec(h)), layer(2, attn))
            # layer 0 runs twice (two caches), layer 2 reads the cache that stop 0 wrote
            schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2, cache_of=0), ScheduleEntry(0))
            return ModelSpec(architecture=self.architecture, vocab_size=r["vocab"], hidden=h, layers=layers,
                             schedule=schedule, final_norm=norm, final_norm_name="norm.weight",
                             embed_name="embed.weight", head_name=None, max_position=512)

    register_architecture(ToyConfig)
    return ToyConfig


def toy_plain(p, raw, ids):
    """The toy model on a whole sequence, in plain tensor arithmetic (64-bit)."""
    t = len(ids)
    x = p["embed.weight"][torch.as_tensor(ids)]
    d, nq, nkv = raw["head_dim"], raw["heads"], raw["kv_heads"]
    cos, sin = pm.rope_tables(torch.arange(t), 100.0, d // 2)
    cos, sin = cos.double(), sin.double()

    def rot(v):          # only the first half of each head is rotated
        return torch.cat([pm.rope_half(v[..., :d // 2], cos, sin), v[..., d // 2:]], -1)

    def qkv(i, h):
        pre = f"blocks.{i}.mixer."
        q = pm.linear(h, p[pre + "q_proj.weight"]).reshape(t, nq, d).transpose(0, 1)
        k = pm.linear(h, p[pre + "k_proj.weight"]).reshape(t, nkv, d).transpose(0, 1)
        v = pm.linear(h, p[pre + "v_proj.weight"]).reshape(t, nkv, d).transpose(0, 1)
        return rot(q), rot(k), v

    def attend(i, q, k, v):
        g = nq // nkv
        k, v = pm.repeat_kv(k, g), pm.repeat_kv(v, g)
        s = torch.matmul(q, k.transpose(1, 2)) / d ** 0.5
        i_ = torch.arange(t)[:, None]
        j_ = torch.arange(t)[None, :]
        s = s.masked_fill((j_ > i_) | (j_ <= i_ - raw["window"]), float("-inf"))
        o = torch.matmul(pm.softmax_last(s), v).transpose(0, 1).reshape(t, nq * d)
        return pm.linear(o, p[f"blocks.{i}.mixer.o_proj.weight"])

    def ffn(i, h):
        pre = f"blocks.{i}.ffn."
        return pm.mlp(h, p[pre + "gate_proj.weight"], p[pre + "up_proj.weight"], p[pre + "down_proj.weight"])

    def norm(name, h):
        return pm.rms_norm(h, p[name], raw["eps"])

    kept = None
    for stop, (layer, reads) in enumerate([(0, None), (1, None), (2, 0), (0, None)]):
        h = norm(f"blocks.{layer}.norm1.weight", x)
        if layer == 1:
            mean = torch.cumsum(h, 0) / torch.arange(1, t + 1, dtype=h.dtype)[:, None]
            a = pm.linear(mean, p["blocks.1.mixer.mix.weight"])
        else:
            q, k, v = qkv(layer, h)
            if stop == 0:
                kept = (k, v)
            if reads is not None:
                k, v = kept
            a = attend(layer, q, k, v)
        x = x + a
        x = x + ffn(layer, norm(f"blocks.{layer}.norm2.weight", x))
    return pm.linear(norm("norm.weight", x), p["embed.weight"])


@pytest.mark.parametrize("dtype,page", [("float32", 4), ("bfloat16", 16)])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype, page):
    from inferrs_amd.engine import Engine, run_trace
    from inferrs_amd.weights import write_random_model
    ToyConfig = register_toy()
    raw = dict(hidden_size=48, heads=4, kv_heads=2, head_dim=16, intermediate=80, vocab=101, eps=1e-5, window=23)
    folder = write_random_model(str(tmp_path / "toy"), ToyConfig(raw), seed=4)
    from safetensors.torch import load_file
    p = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    reqs = {f"r{i}": random_tokens(n, 101, 30 + i) for i, n in enumerate([1, 40, 77, 130])}
    ref = {r: toy_plain(p, raw, t).numpy().astype(np.float32) for r, t in reqs.items()}
    scale = max(float(np.abs(v).max()) for v in ref.values())
    first = None
    for mode, trace in (("whole", tm.whole(reqs)), ("portions", tm.portions(reqs, [5, 2, 31, 3])),
                        ("mixed", tm.mixed(reqs, seed=4, max_live=3, decode_tail=10))):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page) + 2, max_seqs=4)
        assert len(eng.cache.groups) == 1 and len(eng.cache.states) == 1      # two attention caches share a group
        run_trace(eng, trace.lines, str(tmp_path / mode), io.StringIO())
        got = trace.read(str(tmp_path / mode), 101)
        err = max(float(np.abs(got[r][i] - ref[r][i]).max()) for r in reqs for i in range(len(reqs[r]))) / scale
        assert err < (2e-5 if dtype == "float32" else 3e-2), f"{mode}: {err:.3e}"
        eng.cache.check_invariants()
        if first is None:
            first = got
        elif dtype == "float32":
            cross = max(float(np.abs(got[r][i] - first[r][i]).max()) for r in reqs for i in range(len(reqs[r]))) / scale
            assert cross < 2e-6, f"{mode} against whole: {cross:.3e}"


def test_pages_that_a_window_has_passed_may_hold_anything(tmp_path):
    """bfloat16, a window of 23 keys over pages of 16: the matrix-core kernel starts its walk at a multiple of
    32 keys, which may lie in a page that the request has given back.  Every page starts out as NaN here, free
    pages and the one that released table entries name included, and nothing of it reaches the logits."""
    from inferrs_amd.engine import Engine, run_trace
    from inferrs_amd.weights import write_random_model
    ToyConfig = register_toy()
    raw = dict(hidden_size=48, heads=4, kv_heads=2, head_dim=16, intermediate=80, vocab=101, eps=1e-5, window=23)
    folder = write_random_model(str(tmp_path / "toy"), ToyConfig(raw), seed=4)
    from safetensors.torch import load_file
    p = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    reqs = {f"r{i}": random_tokens(n, 101, 130 + i) for i, n in enumerate([61, 40, 150, 97])}
    ref = {r: toy_plain(p, raw, t).numpy().astype(np.float32) for r, t in reqs.items()}
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for mode, trace in (("tail", tm.prefix_then_single(reqs, 40)), ("portions", tm.portions(reqs, [5, 2, 31, 3, 48])),
                        ("mixed", tm.mixed(reqs, seed=6, max_live=3, decode_tail=30))):
        eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=-(-trace.max_tokens // 16) + 2, max_seqs=4)
        for layer in eng.storage.layers.values():
            if layer.k is not None:
                layer.k.fill_(float("nan"))
                layer.v.fill_(float("nan"))
        run_trace(eng, trace.lines, str(tmp_path / mode), io.StringIO())
        got = trace.read(str(tmp_path / mode), 101)
        err = float(np.max([np.abs(got[r][i] - ref[r][i]).max() for r in reqs for i in range(len(reqs[r]))])) / scale
        assert err < 3e-2, f"{mode}: {err:.3e}"             # (numpy's maximum keeps a NaN, and a NaN compares false)


# ---- a second toy architecture: a feed-forward with routing, another position encoding ----------

@dataclass(frozen=True)
class RoutedSpec:
    """A feed-forward that routes: a router scores E experts in 32-bit, the best `top_k` share a token
    by their renormalised softmax weights, and an integer table says which expert's weights stand
    behind a router column.  Expert e: down_e(relu(up_e(h))^2)."""
    hidden: int
    intermediate: int
    experts: int
    top_k: int
    kind: str = "toy_routed"


@dataclass(frozen=True)
class LinearAnglesSpec:
    """A rotary position encoding with another law: angle[p, i] = p * alpha * (i + 1), pairs (2i, 2i+1)."""
    head_dim: int
    rot_dim: int
    alpha: float
    kind: str = "toy_linear_angles"


def register_toy_routed():
    from inferrs_amd import ops
    from inferrs_amd.config import AttentionSpec, LayerSpec, ModelSpec, NormSpec, ScheduleEntry
    from inferrs_amd.config.registry import register_architecture
    from inferrs_amd.parts import FeedForward, Position, register_ffn, register_position
    from inferrs_amd.weights import TensorSpec

    @register_position("toy_linear_angles")
    class LinearAngles(Position):
        interleaved = True

        def __init__(self, spec, tensors, dtype, device):
            self.spec, self.rot_dim = spec, spec.rot_dim
            self.freq = (torch.arange(1, spec.rot_dim // 2 + 1, dtype=torch.float32) * spec.alpha).to(device)

        def table(self, positions):
            angle = positions.to(torch.float32)[:, None] * self.freq[None, :]     # 32-bit, as the rule asks
            return torch.cos(angle).contiguous(), torch.sin(angle).contiguous()

    @register_ffn("toy_routed")
    class Routed(FeedForward):
        @classmethod
        def tensors(cls, spec):
            e = spec.experts
            return {"router.weight": TensorSpec((e, spec.hidden)),
                    "remap": TensorSpec((e,), "table", high=e),
                    "up.weight": TensorSpec((e * spec.intermediate, spec.hidden)),
                    "down.weight": TensorSpec((e * spec.hidden, spec.intermediate))}

        def __init__(self, spec, tensors, dtype, device):
            self.spec = spec
            self.router = tensors["router.weight"].to(device=device, dtype=dtype).contiguous()
            assert tensors["remap"].dtype == torch.int32                    # integer tables stay integers
            self.remap = tensors["remap"].to(device)
            self.up = [w.contiguous() for w in tensors["up.weight"].to(device=device, dtype=dtype).chunk(spec.experts)]
            self.down = [w.contiguous() for w in tensors["down.weight"].to(device=device, dtype=dtype).chunk(spec.experts)]

        def forward(self, ctx, h):
            logits = ops.linear(h, self.router, torch.float32)               # router logits in 32-bit
            best, cols = torch.topk(logits, self.spec.top_k, dim=-1)
            weights = torch.softmax(best, dim=-1)
            out = torch.zeros(h.shape, dtype=torch.float32, device=h.device)
            owner = self.remap[cols]                                         # [n, top_k] expert behind each chosen column
            for e in range(self.spec.experts):
                rows, slot = (owner == e).nonzero(as_tuple=True)
                if rows.numel() == 0:
                    continue
                y = ops.linear(h[rows].contiguous(), self.up[e])
                y = torch.relu(y.float()).square().to(h.dtype)
                out.index_add_(0, rows, ops.linear(y, self.down[e]).float() * weights[rows, slot][:, None])
            return out.to(h.dtype)

    class RoutedConfig:
        architecture = "ToyRoutedForCausalLM"
        model_type = "toy_routed"

        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def to_dict(self):
            return dict(self.raw, architectures=[self.architecture], model_type=self.model_type)

        def to_spec(self):
            r = self.raw
            h = r["hidden_size"]
            norm = NormSpec(size=h, eps=r["eps"])
            attn = AttentionSpec(hidden=h, n_heads=r["heads"], n_kv_heads=r["kv_heads"], head_dim=r["head_dim"],
                                 position=LinearAnglesSpec(r["head_dim"], r["rot_dim"], r["alpha"]), qk_norm=None, window=None)
            ffn = RoutedSpec(h, r["intermediate"], r["experts"], r["top_k"])

            def layer(i):
                p = f"blocks.{i}."
                return LayerSpec(mixer=attn, ffn=ffn, norms=(norm, norm), norm_names=(p + "norm1.weight", p + "norm2.weight"),
                                 mixer_prefix=p + "mixer.", ffn_prefix=p + "ffn.")
            layers = tuple(layer(i) for i in range(r["layers"]))
            return ModelSpec(architecture=self.architecture, vocab_size=r["vocab"], hidden=h, layers=layers,
                             schedule=tuple(ScheduleEntry(i) for i in range(r["layers"])), final_norm=norm,
                             final_norm_name="norm.weight", embed_name="embed.weight", head_name=None, max_position=512)

    register_architecture(RoutedConfig)
    return RoutedConfig


def toy_routed_plain(p, raw, ids):
    """The second toy on a whole sequence in 64-bit: every step written out."""
    t = len(ids)
    x = p["embed.weight"][torch.as_tensor(ids)]
    d, nq, nkv, rot = raw["head_dim"], raw["heads"], raw["kv_heads"], raw["rot_dim"]
    # the engine forms the angles in 32-bit: the plain model takes the same angles, then goes on in 64-bit
    angle = (torch.arange(t, dtype=torch.float32)[:, None] *
             (torch.arange(1, rot // 2 + 1, dtype=torch.float32) * raw["alpha"])[None, :]).double()
    cos, sin = torch.cos(angle), torch.sin(angle)

    def rotate(v):          # pairs (2i, 2i+1) of the first rot features
        a, b = v[..., 0:rot:2], v[..., 1:rot:2]
        out = v.clone()
        out[..., 0:rot:2] = a * cos - b * sin
        out[..., 1:rot:2] = a * sin + b * cos
        return out

    for i in range(raw["layers"]):
        pre = f"blocks.{i}."
        h = pm.rms_norm(x, p[pre + "norm1.weight"], raw["eps"])
        q = rotate(pm.linear(h, p[pre + "mixer.q_proj.weight"]).reshape(t, nq, d).transpose(0, 1))
        k = rotate(pm.linear(h, p[pre + "mixer.k_proj.weight"]).reshape(t, nkv, d).transpose(0, 1))
        v = pm.linear(h, p[pre + "mixer.v_proj.weight"]).reshape(t, nkv, d).transpose(0, 1)
        k, v = pm.repeat_kv(k, nq // nkv), pm.repeat_kv(v, nq // nkv)
        s = torch.matmul(q, k.transpose(1, 2)) / d ** 0.5
        s = s.masked_fill(torch.arange(t)[None, :] > torch.arange(t)[:, None], float("-inf"))
        x = x + pm.linear(torch.matmul(pm.softmax_last(s), v).transpose(0, 1).reshape(t, nq * d), p[pre + "mixer.o_proj.weight"])
        h = pm.rms_norm(x, p[pre + "norm2.weight"], raw["eps"])
        logits = pm.linear(h, p[pre + "ffn.router.weight"])
        best, cols = torch.topk(logits, raw["top_k"], dim=-1)
        weights = pm.softmax_last(best)
        up = p[pre + "ffn.up.weight"].chunk(raw["experts"])
        down = p[pre + "ffn.down.weight"].chunk(raw["experts"])
        remap = p[pre + "ffn.remap"].long()
        y = torch.zeros_like(x)
        for row in range(t):
            for slot in range(raw["top_k"]):
                e = int(remap[cols[row, slot]])
                y[row] += weights[row, slot] * pm.linear(torch.relu(pm.linear(h[row:row + 1], up[e])) ** 2, down[e])[0]
        x = x + y
    return pm.linear(pm.rms_norm(x, p["norm.weight"], raw["eps"]), p["embed.weight"])


@pytest.mark.parametrize("dtype,page,top_k", [("float32", 8, 2), ("bfloat16", 16, 4)])
def test_toy_routed_feed_forward_and_position_encoding(tmp_path, dtype, page, top_k):
    """A feed-forward with routing, a position encoding with another law and an integer table, all
    defined in this file.  In bfloat16 every expert takes part (top_k = experts): a choice among
    experts is not continuous, and rounding may choose otherwise than 64-bit arithmetic does."""
    from inferrs_amd.engine import Engine, run_trace
    from inferrs_amd.weights import write_random_model
    RoutedConfig = register_toy_routed()
    raw = dict(hidden_size=40, heads=5, kv_heads=1, head_dim=16, rot_dim=12, alpha=0.37, intermediate=56, vocab=89,
               eps=1e-4, layers=2, experts=4, top_k=top_k)
    folder = write_random_model(str(tmp_path / "routed"), RoutedConfig(raw), seed=9)
    from safetensors.torch import load_file
    loaded = load_file(os.path.join(folder, "model.safetensors"))
    assert loaded["blocks.0.ffn.remap"].dtype == torch.int32 and int(loaded["blocks.0.ffn.remap"].max()) < 4
    p = {k: (v if v.dtype == torch.int32 else v.double()) for k, v in loaded.items()}
    reqs = {f"r{i}": random_tokens(n, 89, 60 + i) for i, n in enumerate([2, 37, 90])}
    ref = {r: toy_routed_plain(p, raw, t).numpy().astype(np.float32) for r, t in reqs.items()}
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for mode, trace in (("whole", tm.whole(reqs)), ("portions", tm.portions(reqs, [7, 2, 19])),
                        ("mixed", tm.mixed(reqs, seed=5, max_live=3, decode_tail=8))):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page) + 2, max_seqs=4)
        assert not eng.model.graph_safe                 # the toy parts did not say that they can be captured
        run_trace(eng, trace.lines, str(tmp_path / mode), io.StringIO())
        got = trace.read(str(tmp_path / mode), 89)
        err = max(float(np.abs(got[r][i] - ref[r][i]).max()) for r in reqs for i in range(len(reqs[r]))) / scale
        assert err < (2e-5 if dtype == "float32" else 3e-2), f"{mode}: {err:.3e}"
        eng.cache.check_invariants()


@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_of_a_few_rows_with_and_without_the_products_taking_the_norms(tmp_path, name):
    """Steps of up to 12 bfloat16 rows leave the sums into the stream and the norms to the products around
    them; with that switched off the same steps run the norm kernels.  One rounding of a normed value either
    way, at different places: the logits agree to bfloat16's precision, and both agree with the plain model."""
    import plain_model as pm
    from tiny_configs import TINY, random_tokens, write_model
    from inferrs_amd import ops
    from inferrs_amd.engine import Engine, Entry
    raw = TINY[name]
    folder = write_model(str(tmp_path / name), raw, seed=41)
    cfg, params = pm.read_model(folder)
    prompts = {f"r{i}": random_tokens(n, raw["vocab_size"], 700 + i) for i, n in enumerate([9, 5, 11])}
    want = {r: pm.forward(cfg, params, t) for r, t in prompts.items()}
    outs = {}
    for most in (12, 0):
        saved, ops.STREAM_MAX_ROWS = ops.STREAM_MAX_ROWS, most
        try:
            eng = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=16, max_seqs=4)
            rows = [eng.step([Entry(r, t[:4], [3]) for r, t in prompts.items()])]           # 12 rows in one step
            for i in range(4, 9):                                                           # then three rows a step
                rows.append(eng.step([Entry(r, [t[i]], [0]) for r, t in prompts.items() if i < len(t)]))
            outs[most] = rows
        finally:
            ops.STREAM_MAX_ROWS = saved
    scale = max(float(w.abs().max()) for w in want.values())
    for a, b in zip(outs[12], outs[0]):
        assert float((a - b).abs().max()) <= 2e-2 * scale
    for most in (12, 0):
        first = outs[most][0].cpu()
        for j, (r, t) in enumerate(prompts.items()):
            assert float((first[j] - want[r][3]).abs().max()) <= 3e-2 * scale, (most, r)


# ---- a third toy architecture: other ends, another arrangement, values wider than keys -------------

@dataclass(frozen=True)
class WideValueSpec:
    """One-head causal attention without position encoding whose values (dv) are wider than its keys (dk), kept as rows."""
    hidden: int
    dk: int
    dv: int
    kind: str = "toy_wide_value"


@dataclass(frozen=True)
class ScaledEmbeddingSpec:
    vocab_size: int
    hidden: int
    name: str
    scale: float
    kind: str = "toy_scaled_embedding"


@dataclass(frozen=True)
class CappedHeadSpec:
    vocab_size: int
    hidden: int
    cap: float
    kind: str = "toy_capped_head"


def register_toy_ends():
    from inferrs_amd import ops
    from inferrs_amd.config import GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, ScheduleEntry
    from inferrs_amd.config.registry import register_architecture
    from inferrs_amd.parts import (BlockBase, Embedding, Head, Mixer, PagedKV, register_block, register_embedding,
                                   register_head, register_mixer)
    from inferrs_amd.parts.block import build_parts, normed, part_tensors
    from inferrs_amd.weights import TensorSpec

    @register_mixer("toy_wide_value")
    class WideValue(Mixer):
        @classmethod
        def tensors(cls, spec):
            return {"q.weight": TensorSpec((spec.dk, spec.hidden)), "k.weight": TensorSpec((spec.dk, spec.hidden)),
                    "v.weight": TensorSpec((spec.dv, spec.hidden)), "o.weight": TensorSpec((spec.hidden, spec.dv))}

        @classmethod
        def cache_need(cls, spec):
            return PagedKV(1, spec.dk, None, v_head_dim=spec.dv, value_layout="rows")

        def __init__(self, spec, tensors, dtype, device):
            self.spec = spec
            self.w = {n: tensors[n + ".weight"].to(device=device, dtype=dtype).contiguous() for n in "qkvo"}

        def forward(self, ctx, h, cache):
            s = self.spec
            q, k, v = (ops.linear(h, self.w[n]) for n in "qkv")
            group = ctx.groups[cache.group]
            ps = group.page_size
            # (this mixer asked for its values as rows, [page][head][slot][dim], not transposed as the package's own kernels want them)
            assert tuple(cache.k.shape[1:]) == (1, ps, s.dk) and tuple(cache.v.shape[1:]) == (1, ps, s.dv)
            slots = group.slots.long()
            cache.k[slots // ps, 0, slots % ps] = k
            cache.v[slots // ps, 0, slots % ps] = v
            out = torch.empty((h.shape[0], s.dv), dtype=h.dtype, device=h.device)
            off = 0
            for row, (n, start) in enumerate(zip(ctx.q_lens, ctx.kv_starts)):      # a toy: one request at a time
                total = start + n
                pages = group.block_table[row, :-(-total // ps)].long()
                keys = cache.k[pages, 0].reshape(-1, s.dk)[:total].float()
                values = cache.v[pages, 0].reshape(-1, s.dv)[:total].float()
                scores = q[off:off + n].float() @ keys.T / s.dk ** 0.5
                seen = torch.arange(total, device=h.device)[None, :] <= (start + torch.arange(n, device=h.device))[:, None]
                out[off:off + n] = (torch.softmax(scores.masked_fill(~seen, float("-inf")), -1) @ values).to(h.dtype)
                off += n
            return ops.linear(out, self.w["o"])

    @register_block("toy_sandwich")
    class Sandwich(BlockBase):
        """x += post_1(mixer(pre_1(x)));  x += post_2(ffn(pre_2(x))): four norms."""

        @classmethod
        def tensors(cls, spec):
            return part_tensors(spec, 4)

        def __init__(self, spec, tensors, dtype, device):
            self.mixer, self.ffn, self.norms = build_parts(spec, tensors, dtype, device)
            self.first_norm = self.norms[0]

        def parts(self):
            return [self.mixer, self.ffn, *self.norms]

        def forward(self, ctx, x, pending, cache, next_norm=None):
            ctx.stream = ctx.stream_norm = None
            h = normed(self.norms[0], x, pending)
            a = self.norms[1].forward(self.mixer.forward(ctx, h, cache))
            h2 = self.norms[2].add_forward(x, a)
            return x, self.norms[3].forward(self.ffn.forward(ctx, h2))

    @register_embedding("toy_scaled_embedding")
    class ScaledEmbedding(Embedding):
        @classmethod
        def tensors(cls, spec):
            return {spec.name: TensorSpec((spec.vocab_size, spec.hidden))}

        def __init__(self, spec, tensors, dtype, device):
            self.spec = spec
            self.table = tensors[spec.name].to(device=device, dtype=dtype).contiguous()

        def forward(self, ctx):
            return (ops.embed_gather(self.table, ctx.token_ids).float() * self.spec.scale).to(self.table.dtype)

    @register_head("toy_capped_head")
    class CappedHead(Head):
        def __init__(self, spec, tensors, dtype, device, embedding=None):
            self.spec, self.table = spec, embedding.table

        def forward(self, rows):
            logits = ops.linear(rows, self.table, torch.float32)
            return torch.tanh(logits / self.spec.cap) * self.spec.cap

    class EndsConfig:
        architecture = "ToyEndsForCausalLM"
        model_type = "toy_ends"

        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def to_dict(self):
            return dict(self.raw, architectures=[self.architecture], model_type=self.model_type)

        def to_spec(self):
            r = self.raw
            h = r["hidden_size"]
            norm = NormSpec(size=h, eps=r["eps"])
            mixer = WideValueSpec(h, r["dk"], r["dv"])
            ffn = GatedMlpSpec(hidden=h, intermediate=r["intermediate"])

            def layer(i):
                p = f"blocks.{i}."
                return LayerSpec(mixer=mixer, ffn=ffn, norms=(norm,) * 4,
                                 norm_names=tuple(p + f"norm{j}.weight" for j in range(4)),
                                 mixer_prefix=p + "mixer.", ffn_prefix=p + "ffn.", arrangement="toy_sandwich")
            return ModelSpec(architecture=self.architecture, vocab_size=r["vocab"], hidden=h,
                             layers=tuple(layer(i) for i in range(r["layers"])),
                             schedule=tuple(ScheduleEntry(i) for i in range(r["layers"])),
                             final_norm=None, final_norm_name=None, embed_name="embed.weight", head_name=None,
                             max_position=512,
                             embedding=ScaledEmbeddingSpec(r["vocab"], h, "embed.weight", r["embed_scale"]),
                             head=CappedHeadSpec(r["vocab"], h, r["cap"]))

    register_architecture(EndsConfig)
    return EndsConfig


def toy_ends_plain(p, raw, ids):
    t = len(ids)
    x = p["embed.weight"][torch.as_tensor(ids)] * raw["embed_scale"]
    causal = torch.arange(t)[None, :] > torch.arange(t)[:, None]
    for i in range(raw["layers"]):
        pre = f"blocks.{i}."
        norm = lambda j, v: pm.rms_norm(v, p[pre + f"norm{j}.weight"], raw["eps"])
        h = norm(0, x)
        q, k, v = (pm.linear(h, p[pre + f"mixer.{n}.weight"]) for n in "qkv")
        s = (q @ k.T / raw["dk"] ** 0.5).masked_fill(causal, float("-inf"))
        x = x + norm(1, pm.linear(pm.softmax_last(s) @ v, p[pre + "mixer.o.weight"]))
        x = x + norm(3, pm.mlp(norm(2, x), p[pre + "ffn.gate_proj.weight"], p[pre + "ffn.up_proj.weight"],
                               p[pre + "ffn.down_proj.weight"]))
    return torch.tanh(pm.linear(x, p["embed.weight"]) / raw["cap"]) * raw["cap"]


@pytest.mark.parametrize("dtype,page", [("float32", 4), ("bfloat16", 16)])
def test_toy_ends_arrangement_and_unequal_key_and_value_widths(tmp_path, dtype, page):
    """An embedding that scales, a head that caps its logits, no final norm, a block of another arrangement with
    four norms, and a mixer whose cached values are wider than its keys: registered and run from this file."""
    from inferrs_amd.engine import Engine, run_trace
    from inferrs_amd.weights import write_random_model
    EndsConfig = register_toy_ends()
    raw = dict(hidden_size=40, dk=12, dv=28, intermediate=56, vocab=77, eps=1e-5, layers=2, embed_scale=40 ** 0.5, cap=3.0)
    folder = write_random_model(str(tmp_path / "ends"), EndsConfig(raw), seed=6)
    from safetensors.torch import load_file
    loaded = load_file(os.path.join(folder, "model.safetensors"))
    assert "norm.weight" not in loaded and sum(n.startswith("blocks.0.norm") for n in loaded) == 4
    p = {k: v.double() for k, v in loaded.items()}
    reqs = {f"r{i}": random_tokens(n, 77, 80 + i) for i, n in enumerate([3, 29, 70])}
    ref = {r: toy_ends_plain(p, raw, t).numpy().astype(np.float32) for r, t in reqs.items()}
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for mode, trace in (("whole", tm.whole(reqs)), ("portions", tm.portions(reqs, [5, 2, 17])),
                        ("mixed", tm.mixed(reqs, seed=8, max_live=3, decode_tail=6))):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page) + 2, max_seqs=4)
        need = eng.cache.groups[0].need
        assert need.head_dim == 12 and need.value_dim == 28 and len(eng.storage.arrays) == 2
        run_trace(eng, trace.lines, str(tmp_path / mode), io.StringIO())
        got = trace.read(str(tmp_path / mode), 77)
        err = max(float(np.abs(got[r][i] - ref[r][i]).max()) for r in reqs for i in range(len(reqs[r]))) / scale
        assert err < (2e-5 if dtype == "float32" else 3e-2), f"{mode}: {err:.3e}"
        eng.cache.check_invariants()


# ---- a fourth toy architecture: biases on every projection, another activation in the gate -------------

def register_toy_biased():
    from inferrs_amd.config import AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec, ScheduleEntry
    from inferrs_amd.config.registry import register_architecture

    class BiasedConfig:
        architecture = "ToyBiasedForCausalLM"
        model_type = "toy_biased"

        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def to_dict(self):
            return dict(self.raw, architectures=[self.architecture], model_type=self.model_type)

        def to_spec(self):
            r = self.raw
            h, d = r["hidden_size"], r["head_dim"]
            norm = NormSpec(size=h, eps=r["eps"])
            attn = AttentionSpec(hidden=h, n_heads=r["heads"], n_kv_heads=r["kv_heads"], head_dim=d,
                                 position=PositionSpec(kind="rope", head_dim=d, rot_dim=d, theta=1e4),
                                 qk_norm=NormSpec(size=d, eps=r["eps"]), qkv_bias=True, o_bias=True)
            ffn = GatedMlpSpec(hidden=h, intermediate=r["intermediate"], activation="gelu_tanh", bias=True)

            def layer(i):
                p = f"blocks.{i}."
                return LayerSpec(mixer=attn, ffn=ffn, norms=(norm, norm), norm_names=(p + "norm1.weight", p + "norm2.weight"),
                                 mixer_prefix=p + "mixer.", ffn_prefix=p + "ffn.")
            return ModelSpec(architecture=self.architecture, vocab_size=r["vocab"], hidden=h,
                             layers=tuple(layer(i) for i in range(r["layers"])),
                             schedule=tuple(ScheduleEntry(i) for i in range(r["layers"])), final_norm=norm,
                             final_norm_name="norm.weight", embed_name="embed.weight", head_name=None, max_position=512)

    register_architecture(BiasedConfig)
    return BiasedConfig


def gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))


def toy_biased_plain(p, raw, ids):
    t = len(ids)
    x = p["embed.weight"][torch.as_tensor(ids)]
    d, nq, nkv = raw["head_dim"], raw["heads"], raw["kv_heads"]
    cos, sin = pm.rope_tables(torch.arange(t), 1e4, d)
    cos, sin = cos.double(), sin.double()
    causal = torch.arange(t)[None, :] > torch.arange(t)[:, None]
    for i in range(raw["layers"]):
        pre = f"blocks.{i}."
        lin = lambda v, name: pm.linear(v, p[pre + name + ".weight"]) + p[pre + name + ".bias"]
        h = pm.rms_norm(x, p[pre + "norm1.weight"], raw["eps"])
        q = lin(h, "mixer.q_proj").reshape(t, nq, d).transpose(0, 1)
        k = lin(h, "mixer.k_proj").reshape(t, nkv, d).transpose(0, 1)
        v = lin(h, "mixer.v_proj").reshape(t, nkv, d).transpose(0, 1)
        q = pm.rope_half(pm.rms_norm(q, p[pre + "mixer.q_norm.weight"], raw["eps"]), cos, sin)
        k = pm.rope_half(pm.rms_norm(k, p[pre + "mixer.k_norm.weight"], raw["eps"]), cos, sin)
        k, v = pm.repeat_kv(k, nq // nkv), pm.repeat_kv(v, nq // nkv)
        s = (torch.matmul(q, k.transpose(1, 2)) / d ** 0.5).masked_fill(causal, float("-inf"))
        x = x + lin(torch.matmul(pm.softmax_last(s), v).transpose(0, 1).reshape(t, nq * d), "mixer.o_proj")
        h = pm.rms_norm(x, p[pre + "norm2.weight"], raw["eps"])
        x = x + lin(gelu_tanh(lin(h, "ffn.gate_proj")) * lin(h, "ffn.up_proj"), "ffn.down_proj")
    return pm.linear(pm.rms_norm(x, p["norm.weight"], raw["eps"]), p["embed.weight"])


@pytest.mark.parametrize("dtype,page,sizes", [("float32", 4, (48, 4, 2, 16, 80)), ("bfloat16", 16, (48, 4, 2, 16, 80)),
                                              ("bfloat16", 16, (128, 4, 2, 64, 256))])
def test_toy_biases_and_another_gate_activation(tmp_path, dtype, page, sizes):
    """Attention whose four projections have biases and a gated feed-forward with biases and GELU (tanh form) in the
    gate, from the framework's own parts by their specs alone.  The second bfloat16 case has widths in steps of 128 and
    head size 64: decode steps keep the fused attention kernel and the products that take over the stream's sums and
    norms (the bias goes into their sums), and its steps of 17 to 64 rows run the products made for them with the
    bias added behind."""
    from call_counter import CallCounter
    from inferrs_amd.engine import Engine, run_trace
    from inferrs_amd.weights import write_random_model
    BiasedConfig = register_toy_biased()
    hidden, heads, kv_heads, head_dim, inter = sizes
    raw = dict(hidden_size=hidden, heads=heads, kv_heads=kv_heads, head_dim=head_dim, intermediate=inter, vocab=97,
               eps=1e-5, layers=2)
    folder = write_random_model(str(tmp_path / "biased"), BiasedConfig(raw), seed=12)
    from safetensors.torch import load_file, save_file
    loaded = load_file(os.path.join(folder, "model.safetensors"))
    assert loaded["blocks.1.mixer.k_proj.bias"].shape == (kv_heads * head_dim,) and "blocks.0.ffn.down_proj.bias" in loaded
    # biases as large as the products they are added to, so that a lost or misplaced one shows
    for name in loaded:
        if name.endswith(".bias"):
            loaded[name] = (loaded[name].float() * 20).to(loaded[name].dtype)
    save_file(loaded, os.path.join(folder, "model.safetensors"))
    p = {k: v.double() for k, v in loaded.items()}
    reqs = {f"r{i}": random_tokens(n, 97, 90 + i) for i, n in enumerate([3, 21, 45, 70])}
    ref = {r: toy_biased_plain(p, raw, t).numpy().astype(np.float32) for r, t in reqs.items()}
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for mode, trace in (("whole", tm.whole(reqs)), ("tail", tm.prefix_then_single(reqs, 12)),
                        ("portions", tm.portions(reqs, [5, 2, 19, 33])), ("mixed", tm.mixed(reqs, seed=3, max_live=4, decode_tail=9))):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page) + 2, max_seqs=4)
        assert eng.model.graph_safe
        assert bool(eng.load_notes) == (dtype == "bfloat16" and head_dim % 64 != 0)     # off the fused decode kernel: said once
        with CallCounter("attention_decode_fused", "_stream_product", "add_bias") as counted:
            run_trace(eng, trace.lines, str(tmp_path / mode), io.StringIO())
        if dtype == "bfloat16" and head_dim == 64 and mode == "tail":
            assert counted.calls["attention_decode_fused"] > 0 and counted.calls["_stream_product"] > 0, counted.calls
            assert eng.graph_replays > 0
        if dtype == "float32" or mode == "portions":
            assert counted.calls["add_bias"] > 0
        got = trace.read(str(tmp_path / mode), 97)
        err = max(float(np.abs(got[r][i] - ref[r][i]).max()) for r in reqs for i in range(len(reqs[r]))) / scale
        assert err < (2e-5 if dtype == "float32" else 3e-2), f"{mode}: {err:.3e}"
        eng.cache.check_invariants()


def test_an_activation_without_a_kernel_is_refused_by_name():
    from inferrs_amd.config import GatedMlpSpec, SpecError
    from inferrs_amd.parts import part_class
    spec = GatedMlpSpec(hidden=8, intermediate=8, activation="relu")
    with pytest.raises(SpecError, match="relu.*gelu_tanh.*silu"):
        part_class("ffn", spec)(spec, {}, torch.float32, DEV)


# ---- a fifth toy architecture: a mixer that caches one latent row a position, in a paged array of its own ----------

@dataclass(frozen=True)
class LatentSpec:
    """Causal attention over one cached row a position: c = W_c h is what the cache holds (no value array); a query
    q = W_q h scores the rows, and the output is W_o . (softmax(q . c^T / sqrt(dl)) @ c)."""
    hidden: int
    latent: int
    kind: str = "toy_latent"


def register_toy_latent():
    from inferrs_amd import ops
    from inferrs_amd.config import GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, ScheduleEntry
    from inferrs_amd.config.registry import register_architecture
    from inferrs_amd.parts import Mixer, PagedKV, register_mixer
    from inferrs_amd.weights import TensorSpec

    @register_mixer("toy_latent")
    class Latent(Mixer):
        @classmethod
        def tensors(cls, spec):
            return {"c.weight": TensorSpec((spec.latent, spec.hidden)), "q.weight": TensorSpec((spec.latent, spec.hidden)),
                    "o.weight": TensorSpec((spec.hidden, spec.latent))}

        @classmethod
        def cache_need(cls, spec):
            return PagedKV(1, spec.latent, None, values=False)

        def __init__(self, spec, tensors, dtype, device):
            self.spec = spec
            self.w = {n: tensors[n + ".weight"].to(device=device, dtype=dtype).contiguous() for n in "cqo"}

        def forward(self, ctx, h, cache):
            s = self.spec
            assert cache.v is None                                   # one array a layer: the rows'
            c, q = ops.linear(h, self.w["c"]), ops.linear(h, self.w["q"])
            group = ctx.groups[cache.group]
            ps = group.page_size
            slots = group.slots.long()
            cache.k[slots // ps, 0, slots % ps] = c
            out = torch.empty_like(c)
            off = 0
            for row, (n, start) in enumerate(zip(ctx.q_lens, ctx.kv_starts)):      # a toy: one request at a time
                total = start + n
                pages = group.block_table[row, :-(-total // ps)].long()
                rows = cache.k[pages, 0].reshape(-1, s.latent)[:total].float()
                scores = q[off:off + n].float() @ rows.T / s.latent ** 0.5
                seen = torch.arange(total, device=h.device)[None, :] <= (start + torch.arange(n, device=h.device))[:, None]
                out[off:off + n] = (torch.softmax(scores.masked_fill(~seen, float("-inf")), -1) @ rows).to(h.dtype)
                off += n
            return ops.linear(out, self.w["o"])

    class LatentConfig:
        architecture = "ToyLatentForCausalLM"
        model_type = "toy_latent"

        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def to_dict(self):
            return dict(self.raw, architectures=[self.architecture], model_type=self.model_type)

        def to_spec(self):
            r = self.raw
            h = r["hidden_size"]
            norm = NormSpec(size=h, eps=r["eps"])

            def layer(i):
                p = f"blocks.{i}."
                return LayerSpec(mixer=LatentSpec(h, r["latent"]), ffn=GatedMlpSpec(hidden=h, intermediate=r["intermediate"]),
                                 norms=(norm, norm), norm_names=(p + "norm1.weight", p + "norm2.weight"),
                                 mixer_prefix=p + "mixer.", ffn_prefix=p + "ffn.")
            return ModelSpec(architecture=self.architecture, vocab_size=r["vocab"], hidden=h,
                             layers=tuple(layer(i) for i in range(r["layers"])),
                             schedule=tuple(ScheduleEntry(i) for i in range(r["layers"])), final_norm=norm,
                             final_norm_name="norm.weight", embed_name="embed.weight", head_name=None, max_position=512)

    register_architecture(LatentConfig)
    return LatentConfig


def toy_latent_plain(p, raw, ids):
    t = len(ids)
    x = p["embed.weight"][torch.as_tensor(ids)]
    causal = torch.arange(t)[None, :] > torch.arange(t)[:, None]
    for i in range(raw["layers"]):
        pre = f"blocks.{i}."
        h = pm.rms_norm(x, p[pre + "norm1.weight"], raw["eps"])
        c, q = pm.linear(h, p[pre + "mixer.c.weight"]), pm.linear(h, p[pre + "mixer.q.weight"])
        s = (q @ c.T / raw["latent"] ** 0.5).masked_fill(causal, float("-inf"))
        x = x + pm.linear(pm.softmax_last(s) @ c, p[pre + "mixer.o.weight"])
        x = x + pm.mlp(pm.rms_norm(x, p[pre + "norm2.weight"], raw["eps"]), p[pre + "ffn.gate_proj.weight"],
                       p[pre + "ffn.up_proj.weight"], p[pre + "ffn.down_proj.weight"])
    return pm.linear(pm.rms_norm(x, p["norm.weight"], raw["eps"]), p["embed.weight"])


@pytest.mark.parametrize("dtype,page", [("float32", 4), ("bfloat16", 16)])
def test_toy_mixer_with_one_cached_array(tmp_path, dtype, page):
    """A mixer whose paged cache is one array a layer (no values): the storage gives it that and nothing else."""
    from inferrs_amd.engine import Engine, run_trace
    from inferrs_amd.weights import write_random_model
    LatentConfig = register_toy_latent()
    raw = dict(hidden_size=40, latent=24, intermediate=56, vocab=83, eps=1e-5, layers=2)
    folder = write_random_model(str(tmp_path / "latent"), LatentConfig(raw), seed=7)
    from safetensors.torch import load_file
    p = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    reqs = {f"r{i}": random_tokens(n, 83, 40 + i) for i, n in enumerate([2, 33, 71])}
    ref = {r: toy_latent_plain(p, raw, t).numpy().astype(np.float32) for r, t in reqs.items()}
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for mode, trace in (("whole", tm.whole(reqs)), ("portions", tm.portions(reqs, [5, 2, 17])),
                        ("mixed", tm.mixed(reqs, seed=2, max_live=3, decode_tail=6))):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page) + 2, max_seqs=4)
        need = eng.cache.groups[0].need
        assert not need.values and need.value_dim == 0 and len(eng.storage.arrays) == 1
        assert eng.storage.arrays[0].shape[1:] == (eng.cache.groups[0].pool.num_pages, 1, page, 24)
        per_page = 2 * 24 * page * (4 if dtype == "float32" else 2)                  # two layers, one row of 24 a slot
        from inferrs_amd.cache import CacheStorage
        assert CacheStorage.page_bytes(eng.cache, eng.model.dtype) == per_page
        run_trace(eng, trace.lines, str(tmp_path / mode), io.StringIO())
        got = trace.read(str(tmp_path / mode), 83)
        err = max(float(np.abs(got[r][i] - ref[r][i]).max()) for r in reqs for i in range(len(reqs[r]))) / scale
        assert err < (2e-5 if dtype == "float32" else 3e-2), f"{mode}: {err:.3e}"
        eng.cache.check_invariants()


def test_position_part_with_a_scaling_law():
    """`PositionSpec.scaling`: ("linear", f) reads positions as position / f, so the angles at position f * p are
    those of position p without it; a law without an entry is refused by name."""
    from inferrs_amd.config import PositionSpec, SpecError
    from inferrs_amd.parts import part_class
    plain = PositionSpec(kind="rope", head_dim=32, rot_dim=32, theta=1e4)
    scaled = PositionSpec(kind="rope", head_dim=32, rot_dim=32, theta=1e4, scaling=("linear", 4.0))
    a = part_class("position", plain)(plain, {}, torch.float32, DEV)
    b = part_class("position", scaled)(scaled, {}, torch.float32, DEV)
    pos = torch.tensor([0, 1, 5, 300], dtype=torch.int32)
    cos_a, sin_a = a.table(pos.to(DEV))
    cos_b, sin_b = b.table((pos * 4).to(DEV))
    assert float((cos_a - cos_b).abs().max()) < 1e-6 and float((sin_a - sin_b).abs().max()) < 1e-6
    assert torch.equal(b.inv_freq.cpu(), a.inv_freq.cpu() / 4)
    other = PositionSpec(kind="rope", head_dim=32, rot_dim=32, theta=1e4, scaling=("yarn", 4.0))
    with pytest.raises(SpecError, match="yarn.*linear"):
        part_class("position", other)(other, {}, torch.float32, DEV)
