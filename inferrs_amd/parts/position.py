"""Position encodings.  "rope": angle[p, i] = p * theta**(-2i/rot_dim), computed in 32-bit
(`inferrs-models/src/models/attention_utils.rs:186-216`); "none": nothing."""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

from .. import ops
from ..config.spec import PositionSpec, SpecError
from .base import Position, register_position


def inverse_frequencies(theta: float, rot_dim: int) -> np.ndarray:
    """1 / theta**(2i/rot_dim) for i in 0..rot_dim/2 as the reference computes it
    (`attention_utils.rs:198-203`): the exponent, the power and the quotient are 32-bit
    operations.  The power is taken in 64-bit and rounded once, which is what a correctly
    rounded `powf` returns."""
    i = np.arange(rot_dim // 2, dtype=np.float32)
    exponent = (np.float32(2.0) * i) / np.float32(rot_dim)
    power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)
    return (np.float32(1.0) / power).astype(np.float32)


def linear_scaling(inv_freq: np.ndarray, factor: float) -> np.ndarray:
    """Positions read as position / factor: every frequency divided by it, in 32-bit."""
    if not (factor > 0.0):
        raise SpecError(f"rotary scaling 'linear' needs a positive factor, got {factor}")
    return (inv_freq / np.float32(factor)).astype(np.float32)


# name of a scaling law -> (inverse frequencies, factor) -> inverse frequencies; another law is another entry
SCALING_LAWS = {"linear": linear_scaling}


@register_position("rope")
class Rotary(Position):
    graph_safe = True

    def __init__(self, spec: PositionSpec, tensors, dtype, device):
        if spec.rot_dim <= 0 or spec.rot_dim % 2 or spec.rot_dim > spec.head_dim:
            raise SpecError(f"rot_dim {spec.rot_dim} must be even and within head_dim {spec.head_dim}")
        if spec.pairing not in ("half", "interleaved"):
            raise SpecError(f"unknown rotary pairing {spec.pairing!r}")
        self.spec = spec
        self.rot_dim = spec.rot_dim
        self.interleaved = spec.pairing == "interleaved"
        inv_freq = inverse_frequencies(spec.theta, spec.rot_dim)
        if spec.scaling is not None:
            law, factor = spec.scaling
            if law not in SCALING_LAWS:
                raise SpecError(f"rotary scaling {law!r} has no entry (known: {sorted(SCALING_LAWS)})")
            inv_freq = SCALING_LAWS[law](inv_freq, float(factor))
        self.inv_freq = torch.from_numpy(inv_freq).to(device)

    def table(self, positions: torch.Tensor) -> Optional[Tuple[torch.Tensor, torch.Tensor]]:
        return ops.rope_table(positions, self.inv_freq)


@register_position("none")
class NoPosition(Position):
    graph_safe = True

    rot_dim = 0
    interleaved = False

    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec

    def table(self, positions):
        return None
