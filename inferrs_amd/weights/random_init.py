"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no random-weight mode for this model (candle's
`VarBuilder::zeros` exists, `candle-nn/src/var_builder.rs:616`, unused).  Each
tensor has a seed of its own from (seed, tensor name) and each element is a
function of (that seed, its index) alone, so values do not depend on which other
tensors exist, on the order of filling or on where they are filled (host or
GPU): matrices N(0, 0.02), norm weights 1 + N(0, 0.1), rounded to 32-bit and
then to the storage precision.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Mapping

import numpy as np
import torch

from .loader import TensorSpec
from .safetensors_io import write_safetensors

MATRIX_STD = 0.02
NORM_STD = 0.1


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little") & (2**63 - 1)


_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _splitmix_out(state: np.ndarray) -> np.ndarray:
    z = state
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def normal_values(n: int, seed: int, mean: float, std: float) -> np.ndarray:
    """float32 [n]: element i is mean + std * z_i, z_i standard normal by Box and Muller from two
    outputs of the splitmix64 sequence started at seed + 2 i steps, all in 64-bit arithmetic.  The
    device kernel `ia_fill_normal` computes the same."""
    out = np.empty(n, dtype=np.float32)
    step = 1 << 22
    with np.errstate(over="ignore"):
        for lo in range(0, n, step):
            i = np.arange(lo, min(n, lo + step), dtype=np.uint64)
            base = np.uint64(seed & (2**64 - 1))
            h1 = _splitmix_out(base + (np.uint64(2) * i + np.uint64(1)) * _GOLDEN)
            h2 = _splitmix_out(base + (np.uint64(2) * i + np.uint64(2)) * _GOLDEN)
            u1 = ((h1 >> np.uint64(11)) + np.uint64(1)).astype(np.float64) * (1.0 / 9007199254740992.0)
            u2 = (h2 >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
            z = np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586 * u2)
            out[lo:lo + i.size] = (mean + std * z).astype(np.float32)
    return out


def n_elements(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


def table_values(n: int, seed: int, high: int) -> np.ndarray:
    """int32 [n]: element i is output i + 1 of the splitmix64 sequence started at seed, modulo `high`."""
    with np.errstate(over="ignore"):
        i = np.arange(1, n + 1, dtype=np.uint64)
        h = _splitmix_out(np.uint64(seed & (2**64 - 1)) + i * _GOLDEN)
    return (h % np.uint64(high)).astype(np.int32)


def random_tensors(expected: Mapping[str, TensorSpec], seed: int,
                   dtype: torch.dtype = torch.bfloat16,
                   device: str = "cpu") -> Dict[str, torch.Tensor]:
    """Every tensor of `expected`, filled on `device`: on the host with NumPy, on the GPU by
    the fill kernel; both give the same values."""
    on_gpu = torch.device(device).type == "cuda"
    if on_gpu:
        from .. import ops
    out: Dict[str, torch.Tensor] = {}
    for name, spec in expected.items():
        if spec.init == "table":
            if spec.high <= 0:
                raise ValueError(f"no random fill is defined for integer table '{name}' (its TensorSpec gives no range)")
            out[name] = torch.from_numpy(table_values(n_elements(spec.shape), _tensor_seed(seed, name), spec.high)
                                         ).reshape(spec.shape).to(device)
            continue
        mean, std = (1.0, NORM_STD) if spec.init == "norm" else (0.0, MATRIX_STD)
        tseed = _tensor_seed(seed, name)
        if on_gpu:
            out[name] = ops.fill_normal(spec.shape, tseed, mean, std, dtype, device)
        else:
            out[name] = torch.from_numpy(normal_values(n_elements(spec.shape), tseed, mean, std)).reshape(spec.shape).to(dtype)
    return out


def write_random_model(model_dir: str, config, seed: int,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write `config.json` and `model.safetensors` for `config` (a registered
    architecture's configuration object) and return the folder."""
    from ..parts.assemble import generated_tensors
    spec = config.to_spec()
    wanted = generated_tensors(spec)
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      random_tensors(wanted, seed, dtype),
                      metadata={"format": "pt", "seed": str(seed)})
    return model_dir
