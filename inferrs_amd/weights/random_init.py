"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no random-weight mode for this model (candle's
`VarBuilder::zeros` exists, `candle-nn/src/var_builder.rs:616`, unused).  Each
tensor is drawn from a generator keyed by (seed, tensor name), so a tensor's
values do not depend on which other tensors exist or on the order of filling:
matrices N(0, 0.02), norm weights 1 + N(0, 0.1), drawn in 32-bit and then
rounded to the storage precision.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Mapping

import torch

from .loader import TensorSpec
from .safetensors_io import write_safetensors

MATRIX_STD = 0.02
NORM_STD = 0.1


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little") & (2**63 - 1)


def random_tensors(expected: Mapping[str, TensorSpec], seed: int,
                   dtype: torch.dtype = torch.bfloat16,
                   device: str = "cpu") -> Dict[str, torch.Tensor]:
    out: Dict[str, torch.Tensor] = {}
    gen = torch.Generator(device=device)
    for name, spec in expected.items():
        gen.manual_seed(_tensor_seed(seed, name))
        if spec.init == "table":
            raise ValueError(f"no random fill is defined for integer table '{name}'")
        t = torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device)
        if spec.init == "norm":
            t.mul_(NORM_STD).add_(1.0)
        else:
            t.mul_(MATRIX_STD)
        out[name] = t.to(dtype)
    return out


def write_random_model(model_dir: str, config, seed: int,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write `config.json` and `model.safetensors` for `config` (a registered
    architecture's configuration object) and return the folder."""
    from ..parts.assemble import model_tensors
    spec = config.to_spec()
    expected, optional = model_tensors(spec)
    wanted = {n: s for n, s in expected.items() if n not in optional}
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      random_tensors(wanted, seed, dtype),
                      metadata={"format": "pt", "seed": str(seed)})
    return model_dir
