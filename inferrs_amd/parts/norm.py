"""RMS norm: x / sqrt(mean(x^2) + eps) * w, statistics in 32-bit
(`candle-nn/src/ops.rs:443-504`, `inferrs-kernels/candle-kernels/src/reduce.cu:189-228`)."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import NormSpec
from ..weights.loader import TensorSpec
from .base import Norm, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    @classmethod
    def tensors(cls, spec: NormSpec) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((spec.size,), "norm")}

    def __init__(self, spec: NormSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec = spec
        self.eps = float(spec.eps)
        self.add_one = bool(spec.add_one)
        # Norm weights are vectors: kept in 32-bit whatever the activations are stored in.
        self.weight = tensors["weight"].to(device=device, dtype=torch.float32).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, self.add_one)

    def add_forward(self, x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, self.add_one)

    def add_forward_partials(self, x: torch.Tensor, delta: "ops.Partials") -> torch.Tensor:
        """`add_forward` for a product that is still split along k."""
        return ops.add_rmsnorm_partials(x, delta, self.weight, self.eps, self.add_one)

    def rows_for_product(self, x: torch.Tensor, added: "ops.Added") -> ops.NormedRows:
        """The norm of a stream's rows left to the product that reads them: `added` holds the rows times
        this norm's weight and their sums of squares."""
        return ops.NormedRows(x, added.scaled, added.sums, self.weight, self.eps, self.add_one)
