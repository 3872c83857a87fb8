"""Gated feed-forward: down( silu(gate(x)) * up(x) ), no biases
(`inferrs-models/src/models/attention_utils.rs:94-118`).  Gate and up share one product."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import GatedMlpSpec, SpecError
from ..weights.loader import TensorSpec
from .base import FeedForward, register_ffn
from .linear import Linear


@register_ffn("gated_mlp")
class GatedMlp(FeedForward):
    graph_safe = True
    takes_normed_rows = True      # the gate|up product norms the rows it is given as `ops.NormedRows`
    adds_to_stream = True         # the down product adds itself to `ctx.stream` where it can

    @classmethod
    def tensors(cls, spec: GatedMlpSpec) -> Dict[str, TensorSpec]:
        return {
            "gate_proj.weight": TensorSpec((spec.intermediate, spec.hidden)),
            "up_proj.weight": TensorSpec((spec.intermediate, spec.hidden)),
            "down_proj.weight": TensorSpec((spec.hidden, spec.intermediate)),
        }

    def __init__(self, spec: GatedMlpSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if spec.activation != "silu":
            raise SpecError(f"gated_mlp: activation {spec.activation!r} has no kernel (only 'silu')")
        self.spec = spec
        self.gate_up = Linear([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dtype, device)
        self.down = Linear([tensors["down_proj.weight"]], dtype, device)

    def forward(self, ctx, h):
        act = ops.gated_silu_linear(h, self.gate_up.weight)
        if getattr(ctx, "stream", None) is not None:
            norm = getattr(ctx, "stream_norm", None)
            added = ops.linear_add(act, self.down.weight, ctx.stream, norm)
            if added is not None:
                return ops.Added(added[0], added[1], norm)
        if getattr(ctx, "partial_sums", False):
            split = ops.linear_partials(act, self.down.weight)
            if split is not None:
                return split
        return self.down(act)
