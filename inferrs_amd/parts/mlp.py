"""Gated feed-forward: down( act(gate(x)) * up(x) ); the reference's is SiLU without biases
(`inferrs-models/src/models/attention_utils.rs:94-118`).  Gate and up share one product; the
activation (a name of `ops.ACTIVATIONS`) and optional biases are the spec's."""
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
        t = {
            "gate_proj.weight": TensorSpec((spec.intermediate, spec.hidden)),
            "up_proj.weight": TensorSpec((spec.intermediate, spec.hidden)),
            "down_proj.weight": TensorSpec((spec.hidden, spec.intermediate)),
        }
        if spec.bias:
            t["gate_proj.bias"] = TensorSpec((spec.intermediate,))
            t["up_proj.bias"] = TensorSpec((spec.intermediate,))
            t["down_proj.bias"] = TensorSpec((spec.hidden,))
        return t

    def __init__(self, spec: GatedMlpSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if spec.activation not in ops.ACTIVATIONS:
            raise SpecError(f"gated_mlp: activation {spec.activation!r} has no kernel (known: {sorted(ops.ACTIVATIONS)})")
        self.spec = spec
        self.gate_up = Linear([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dtype, device,
                              [tensors["gate_proj.bias"], tensors["up_proj.bias"]] if spec.bias else None)
        self.down = Linear([tensors["down_proj.weight"]], dtype, device, [tensors["down_proj.bias"]] if spec.bias else None)

    def forward(self, ctx, h):
        act = ops.gated_linear(h, self.gate_up.weight, self.spec.activation, self.gate_up.bias)
        if getattr(ctx, "stream", None) is not None:
            norm = getattr(ctx, "stream_norm", None)
            added = ops.linear_add(act, self.down.weight, ctx.stream, norm, self.down.bias)
            if added is not None:
                return ops.Added(added[0], added[1], norm)
        if getattr(ctx, "partial_sums", False):
            split = ops.linear_partials(act, self.down.weight, self.down.bias)
            if split is not None:
                return split
        return self.down(act)
