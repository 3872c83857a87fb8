"""A weight matrix [out, in] in the compute precision, applied as x . W^T (+ bias)
(`candle-nn/src/linear.rs:64-72`)."""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from .. import ops


def to_compute(t: torch.Tensor, dtype: torch.dtype, device) -> torch.Tensor:
    """Stored precision -> compute precision.  bfloat16 -> 32-bit is exact; a 32-bit tensor
    used by a bfloat16 model is rounded once here."""
    return t.to(device=device, dtype=dtype).contiguous()


class Linear:
    def __init__(self, weights: Sequence[torch.Tensor], dtype: torch.dtype, device,
                 biases: Optional[Sequence[torch.Tensor]] = None):
        """`weights`: one or more [out_i, in] matrices that share the input; they are stacked
        along `out` so that one product serves all of them.  `biases`: None, or one [out_i] vector
        for each of them, stacked likewise and added to every row of the product."""
        mats = [to_compute(w, dtype, device) for w in weights]
        self.weight = mats[0] if len(mats) == 1 else torch.cat(mats, dim=0).contiguous()
        self.out_features, self.in_features = self.weight.shape
        self.bias = None
        if biases is not None:
            if len(biases) != len(mats) or any(b.numel() != m.shape[0] for b, m in zip(biases, mats)):
                raise ValueError("Linear: one bias of `out` entries for every weight matrix")
            self.bias = torch.cat([to_compute(b, dtype, device).reshape(-1) for b in biases]).contiguous()

    def __call__(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.linear(x, self.weight, out_dtype, bias=self.bias)
