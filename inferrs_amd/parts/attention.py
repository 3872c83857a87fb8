"""Grouped-query attention over the paged cache.

Order of operations as in the reference (`inferrs-models/src/models/qwen3.rs:105-195`):
q, k, v projections without bias; per-head RMS norm of q and k; rotation of q and k by
position; append of k and v to the cache; scores (q.k)/sqrt(d) against keys at positions
<= the query's (and inside the window, when one is set); softmax; weighted sum of values;
output projection.  q head h reads kv head h // (n_heads / n_kv_heads)
(`attention_utils.rs:38-49`).
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import AttentionSpec, SpecError
from ..weights.loader import TensorSpec
from .base import Mixer, PagedKV, part_class, register_mixer
from .linear import Linear


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True
    takes_normed_rows = True      # the q|k|v product norms the rows it is given as `ops.NormedRows`
    adds_to_stream = True         # the output projection adds itself to `ctx.stream` where it can

    @classmethod
    def tensors(cls, spec: AttentionSpec) -> Dict[str, TensorSpec]:
        q_out, kv_out = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim
        t = {
            "q_proj.weight": TensorSpec((q_out, spec.hidden)),
            "k_proj.weight": TensorSpec((kv_out, spec.hidden)),
            "v_proj.weight": TensorSpec((kv_out, spec.hidden)),
            "o_proj.weight": TensorSpec((spec.hidden, q_out)),
        }
        if spec.qk_norm is not None:
            t["q_norm.weight"] = TensorSpec((spec.head_dim,), "norm")
            t["k_norm.weight"] = TensorSpec((spec.head_dim,), "norm")
        if spec.qkv_bias:
            t["q_proj.bias"] = TensorSpec((q_out,))
            t["k_proj.bias"] = TensorSpec((kv_out,))
            t["v_proj.bias"] = TensorSpec((kv_out,))
        if spec.o_bias:
            t["o_proj.bias"] = TensorSpec((spec.hidden,))
        return t

    @classmethod
    def cache_need(cls, spec: AttentionSpec):
        return PagedKV(spec.n_kv_heads, spec.head_dim, spec.window)

    def __init__(self, spec: AttentionSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if spec.n_heads % spec.n_kv_heads:
            raise SpecError(f"attention: {spec.n_heads} heads are not a multiple of {spec.n_kv_heads} kv heads")
        # (the matrix-core kernels take head sizes in steps of 16 up to 256 in bfloat16; every other size, and the
        # 32-bit path, runs on the plain kernels, which take any size up to 512)
        if not (1 <= spec.head_dim <= 512):
            raise SpecError(f"attention: head_dim {spec.head_dim} is outside 1..512, the range of the attention kernels")
        rot = getattr(spec.position, "rot_dim", 0) if getattr(spec.position, "kind", "none") != "none" else 0
        if rot % 2 or rot > spec.head_dim:
            raise SpecError(f"attention: the rotated part of a head ({rot}) must be even and within head_dim {spec.head_dim}")
        if spec.window is not None and spec.window < 1:
            raise SpecError(f"attention: window {spec.window} must be >= 1")
        if spec.qk_norm is not None and spec.qk_norm.size != spec.head_dim:
            raise SpecError("attention: qk_norm must span head_dim")
        self.spec = spec
        self.qkv = Linear([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], dtype, device,
                          [tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]] if spec.qkv_bias else None)
        self.o = Linear([tensors["o_proj.weight"]], dtype, device, [tensors["o_proj.bias"]] if spec.o_bias else None)
        if spec.qk_norm is not None:
            self.q_norm_w = tensors["q_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            self.k_norm_w = tensors["k_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            self.norm_eps, self.norm_add_one = float(spec.qk_norm.eps), bool(spec.qk_norm.add_one)
        else:
            self.q_norm_w = self.k_norm_w = None
            self.norm_eps, self.norm_add_one = 0.0, False
        self.position = part_class("position", spec.position)(spec.position, {}, dtype, device)

    def load_notes(self, page_size: int):
        """What the log should say once when a model with this part is set up: a decode step that cannot take the
        fused kernel still runs, three kernels where one would do."""
        dtype = self.qkv.weight.dtype
        has_rotation = self.position.rot_dim > 0
        if dtype != torch.bfloat16 or ops.attention_decode_fused_fits(dtype, self.spec.head_dim, page_size,
                                                                      self.position.rot_dim, self.position.interleaved,
                                                                      has_rotation):
            return []
        s = self.spec
        return [f"attention with head size {s.head_dim}, page size {page_size}, rotation of {self.position.rot_dim} features "
                f"({'interleaved' if self.position.interleaved else 'halves'}): decode steps do not take the fused kernel "
                "(head sizes in steps of 64, page sizes in steps of 16, whole heads rotated in halves); norm and "
                "rotation, the cache write and the attention run as kernels of their own"]

    def _project(self, ctx, a: torch.Tensor):
        """The output projection: added to the step's stream by the product itself where that can be."""
        if getattr(ctx, "stream", None) is not None:
            norm = getattr(ctx, "stream_norm", None)
            added = ops.linear_add(a, self.o.weight, ctx.stream, norm, self.o.bias)
            if added is not None:
                return ops.Added(added[0], added[1], norm)
        if getattr(ctx, "partial_sums", False):
            split = ops.linear_partials(a, self.o.weight, self.o.bias)
            if split is not None:
                return split
        return self.o(a)

    def forward(self, ctx, h, cache):
        s = self.spec
        group = ctx.groups[cache.group]
        qkv = self.qkv(h)
        table = ctx.position_table(self.position)
        cos, sin = table if table is not None else (None, None)
        if ctx.max_q_len == 1 and ops.attention_decode_fused_fits(qkv.dtype, s.head_dim, group.page_size,
                                                                   self.position.rot_dim, self.position.interleaved,
                                                                   cos is not None):
            # decode steps: norm, rotation, cache write and attention in one kernel
            a = ops.attention_decode_fused(
                qkv, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table, nq=s.n_heads,
                nkv=s.n_kv_heads, d=s.head_dim, slots=group.slots if cache.writable else None,
                q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, eps=self.norm_eps, add_one=self.norm_add_one,
                cos=cos, sin=sin, max_kv_len=ctx.max_kv_len, window=s.window, scale=s.softmax_scale)
            return self._project(ctx, a.view(a.shape[0], s.n_heads * s.head_dim))
        q = ops.qk_rope_kv(
            qkv, s.n_heads, s.n_kv_heads, s.head_dim,
            q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, eps=self.norm_eps, add_one=self.norm_add_one,
            cos=cos, sin=sin, rot=self.position.rot_dim, interleaved=self.position.interleaved,
            k_cache=cache.k, v_cache=cache.v, slots=group.slots if cache.writable else None,
            page_size=group.page_size)
        if ops.attention_mfma_fits(q.dtype, s.head_dim, group.page_size):
            common = dict(window=s.window, scale=s.softmax_scale)
            if 0 < ctx.n_single < ctx.n_seqs:
                # single tokens (decode) and portions of prompts want different launches: the first
                # split their long key ranges between waves, the second have columns enough
                a = ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                       max_q_len=1, max_kv_len=ctx.max_kv_single, seqs=(0, ctx.n_single),
                                       tokens=(0, ctx.n_single), **common)
                ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                   max_q_len=ctx.max_q_len, max_kv_len=ctx.max_kv_multi,
                                   seqs=(ctx.n_single, ctx.n_seqs - ctx.n_single),
                                   tokens=(ctx.n_single, ctx.n_tokens - ctx.n_single), out=a, **common)
            else:
                a = ops.attention_mfma(q, cache.k, cache.v, ctx.positions, ctx.cu_tokens, group.block_table,
                                       max_q_len=ctx.max_q_len, max_kv_len=ctx.max_kv_len, **common)
        else:
            a = ops.attention_generic(q, cache.k, cache.v, ctx.positions, ctx.token_seq, group.block_table,
                                      window=s.window, scale=s.softmax_scale, max_kv_len=ctx.max_kv_len)
        return self._project(ctx, a.view(a.shape[0], s.n_heads * s.head_dim))
