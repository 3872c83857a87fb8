"""One residual block.  Arrangement "pre_norm" as in the reference
(`inferrs-models/src/models/qwen3.rs:284-300`):

    x = x + mixer(norm_0(x));  x = x + ffn(norm_1(x))

The sums are formed in 32-bit inside the norm kernel that follows them, so a block takes
the stream `x` together with the not-yet-added output of the block before it and returns
the same pair.  In steps of a few rows the products around a norm can take over both the sum
and the norm (`ops.Added`, `ops.NormedRows`).

Other arrangements (norms after the parts, four norms around them, parts side by side) are other
classes under `register_block`; the model asks the table by `LayerSpec.arrangement`.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from .. import ops
from ..config.spec import LayerSpec, SpecError
from ..weights.loader import TensorSpec
from .base import BlockBase, part_class, register_block


def sub_tensors(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def part_tensors(layer: LayerSpec, n_norms: int) -> Dict[str, TensorSpec]:
    """The tensors of a layer's mixer, feed-forward and `n_norms` norms, by full name."""
    if len(layer.norms) != n_norms or len(layer.norm_names) != n_norms:
        raise SpecError(f"the arrangement {layer.arrangement!r} has {n_norms} norms, the layer names {len(layer.norms)}")
    out: Dict[str, TensorSpec] = {}
    for local, ts in part_class("mixer", layer.mixer).tensors(layer.mixer).items():
        out[layer.mixer_prefix + local] = ts
    for local, ts in part_class("ffn", layer.ffn).tensors(layer.ffn).items():
        out[layer.ffn_prefix + local] = ts
    for name, nspec in zip(layer.norm_names, layer.norms):
        (ts,) = part_class("norm", nspec).tensors(nspec).values()
        out[name] = ts
    return out


def build_parts(layer: LayerSpec, tensors: Dict[str, torch.Tensor], dtype, device):
    """(mixer, feed-forward, [norms]) of a layer."""
    mixer = part_class("mixer", layer.mixer)(layer.mixer, sub_tensors(tensors, layer.mixer_prefix), dtype, device)
    ffn = part_class("ffn", layer.ffn)(layer.ffn, sub_tensors(tensors, layer.ffn_prefix), dtype, device)
    norms = [part_class("norm", nspec)(nspec, {"weight": tensors[name]}, dtype, device)
             for name, nspec in zip(layer.norm_names, layer.norms)]
    return mixer, ffn, norms


@register_block("pre_norm")
class Block(BlockBase):
    N_NORMS = 2

    @classmethod
    def tensors(cls, spec: LayerSpec) -> Dict[str, TensorSpec]:
        return part_tensors(spec, cls.N_NORMS)

    def __init__(self, spec: LayerSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if len(spec.norms) != self.N_NORMS:
            raise SpecError(f"a pre-norm block has two norms, the layer names {len(spec.norms)}")
        self.spec = spec
        self.mixer, self.ffn, (self.norm_mixer, self.norm_ffn) = build_parts(spec, tensors, dtype, device)
        self.first_norm = self.norm_mixer

    def parts(self):
        return [self.mixer, self.ffn, self.norm_mixer, self.norm_ffn, getattr(self.mixer, "position", None)]

    def forward(self, ctx, x: torch.Tensor, pending, cache, next_norm=None) -> Tuple[torch.Tensor, object]:
        # Steps of a few bfloat16 rows (decode): a part that says `adds_to_stream` may add its output to
        # `ctx.stream` itself and return `ops.Added` instead (the new rows' sums of squares, and the rows
        # times the weight of `ctx.stream_norm`, the norm that comes next: `next_norm` after this block),
        # and a part that says `takes_normed_rows` may get `ops.NormedRows` made of these, whose norm its
        # first product finishes.
        mid_from = ops.mid_from_rows(x.shape[1])
        few = x.dtype == torch.bfloat16 and 0 < x.shape[0] <= min(ops.STREAM_MAX_ROWS, mid_from - 1)
        # Steps of `ops.mid_from_rows(width)` to `ops.MID_MAX_ROWS` bfloat16 rows: a part's last product may stay split along k (`ops.Partials`); the norm
        # that adds it to the stream adds the splits up on the way (`normed` below, or whoever reads `pending`).
        ctx.partial_sums = x.dtype == torch.bfloat16 and mid_from <= x.shape[0] <= ops.MID_MAX_ROWS
        h = normed(self.norm_mixer, x, pending, few and getattr(self.mixer, "takes_normed_rows", False))
        ctx.stream = x if few and getattr(self.mixer, "adds_to_stream", False) else None
        ctx.stream_norm = self.norm_ffn if getattr(self.ffn, "takes_normed_rows", False) else None
        a = self.mixer.forward(ctx, h, cache)
        h2 = normed(self.norm_ffn, x, a, few and getattr(self.ffn, "takes_normed_rows", False))
        ctx.stream = x if few and getattr(self.ffn, "adds_to_stream", False) else None
        ctx.stream_norm = next_norm
        out = self.ffn.forward(ctx, h2)
        ctx.stream = ctx.stream_norm = None
        ctx.partial_sums = False
        return x, out


def settle(x: torch.Tensor, pending) -> torch.Tensor:
    """The stream with `pending` added (in place): for arrangements and model ends that do not begin with a norm."""
    if isinstance(pending, ops.Partials):
        pending = pending.materialize()
    if pending is not None and not isinstance(pending, ops.Added):
        ops.add_inplace(x, pending)
    return x


def normed(norm, x: torch.Tensor, pending, lazy: bool = False):
    """norm(x + pending), the sum left in x; `pending` None: nothing to add; `ops.Partials`: a product still split along k, added
    up by the norm's kernel (or here, for a norm that has none for it); `ops.Added`: x holds the sum
    already, and with `lazy` the norm is left to the product that reads the rows, if the part that added
    them has prepared them for this norm."""
    if pending is None:
        return norm.forward(x)
    if isinstance(pending, ops.Partials):
        if hasattr(norm, "add_forward_partials"):
            return norm.add_forward_partials(x, pending)
        pending = pending.materialize()
    if isinstance(pending, ops.Added):
        if lazy and pending.scaled is not None and pending.norm is norm and hasattr(norm, "rows_for_product"):
            return norm.rows_for_product(x, pending)
        return norm.forward(x)
    return norm.add_forward(x, pending)
