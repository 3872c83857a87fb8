"""One residual block.  Arrangement "pre_norm" as in the reference
(`inferrs-models/src/models/qwen3.rs:284-300`):

    x = x + mixer(norm_mixer(x));  x = x + ffn(norm_ffn(x))

The sums are formed in 32-bit inside the norm kernel that follows them, so a block takes
the stream `x` together with the not-yet-added output of the block before it and returns
the same pair.  In steps of a few rows the products around a norm can take over both the sum
and the norm (`ops.Added`, `ops.NormedRows`).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .. import ops
from ..config.spec import LayerSpec, SpecError
from .base import part_class


class Block:
    def __init__(self, spec: LayerSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if spec.arrangement != "pre_norm":
            raise SpecError(f"unknown block arrangement {spec.arrangement!r}")
        self.spec = spec

        def sub(prefix: str) -> Dict[str, torch.Tensor]:
            return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}

        self.mixer = part_class("mixer", spec.mixer)(spec.mixer, sub(spec.mixer_prefix), dtype, device)
        self.ffn = part_class("ffn", spec.ffn)(spec.ffn, sub(spec.ffn_prefix), dtype, device)
        self.norm_mixer = part_class("norm", spec.norm_mixer)(
            spec.norm_mixer, {"weight": tensors[spec.norm_mixer_name]}, dtype, device)
        self.norm_ffn = part_class("norm", spec.norm_ffn)(
            spec.norm_ffn, {"weight": tensors[spec.norm_ffn_name]}, dtype, device)

    def forward(self, ctx, x: torch.Tensor, pending, cache, next_norm=None) -> Tuple[torch.Tensor, object]:
        # Steps of a few bfloat16 rows (decode): a part that says `adds_to_stream` may add its output to
        # `ctx.stream` itself and return `ops.Added` instead (the new rows' sums of squares, and the rows
        # times the weight of `ctx.stream_norm`, the norm that comes next: `next_norm` after this block),
        # and a part that says `takes_normed_rows` may get `ops.NormedRows` made of these, whose norm its
        # first product finishes.
        few = x.dtype == torch.bfloat16 and 0 < x.shape[0] <= ops.STREAM_MAX_ROWS
        h = normed(self.norm_mixer, x, pending, few and getattr(self.mixer, "takes_normed_rows", False))
        ctx.stream = x if few and getattr(self.mixer, "adds_to_stream", False) else None
        ctx.stream_norm = self.norm_ffn if getattr(self.ffn, "takes_normed_rows", False) else None
        a = self.mixer.forward(ctx, h, cache)
        h2 = normed(self.norm_ffn, x, a, few and getattr(self.ffn, "takes_normed_rows", False))
        ctx.stream = x if few and getattr(self.ffn, "adds_to_stream", False) else None
        ctx.stream_norm = next_norm
        out = self.ffn.forward(ctx, h2)
        ctx.stream = ctx.stream_norm = None
        return x, out


def normed(norm, x: torch.Tensor, pending, lazy: bool = False):
    """norm(x + pending), the sum left in x; `pending` None: nothing to add; `ops.Added`: x holds the sum
    already, and with `lazy` the norm is left to the product that reads the rows, if the part that added
    them has prepared them for this norm."""
    if pending is None:
        return norm.forward(x)
    if isinstance(pending, ops.Added):
        if lazy and pending.scaled is not None and pending.norm is norm and hasattr(norm, "rows_for_product"):
            return norm.rows_for_product(x, pending)
        return norm.forward(x)
    return norm.add_forward(x, pending)
