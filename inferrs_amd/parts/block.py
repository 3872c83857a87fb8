"""One residual block.  Arrangement "pre_norm" as in the reference
(`inferrs-models/src/models/qwen3.rs:284-300`):

    x = x + mixer(norm_mixer(x));  x = x + ffn(norm_ffn(x))

The sums are formed in 32-bit inside the norm kernel that follows them, so a block takes
the stream `x` together with the not-yet-added output of the block before it and returns
the same pair.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

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

    def forward(self, ctx, x: torch.Tensor, pending: Optional[torch.Tensor],
                cache) -> Tuple[torch.Tensor, torch.Tensor]:
        h = self.norm_mixer.forward(x) if pending is None else self.norm_mixer.add_forward(x, pending)
        a = self.mixer.forward(ctx, h, cache)
        h2 = self.norm_ffn.add_forward(x, a)
        return x, self.ffn.forward(ctx, h2)
