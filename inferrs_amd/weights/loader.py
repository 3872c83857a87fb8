"""Weights by tensor name, checked against what the model's parts expect.

The reference reads each tensor eagerly by name and fails on the first one
that is missing (`CannotFindTensor`, `candle-core/src/safetensors.rs:501-515`)
or has another shape (`shape mismatch for {name}`,
`candle-nn/src/var_builder.rs:509-518`).  Here the whole folder is checked
first and ONE error lists every missing tensor and every wrong shape, so a bad
checkpoint is diagnosed in one go; it lists the tensors that the model does not
read as well ("unexpected tensors"), since a misnamed tensor is one missing and one
unexpected.  Such tensors alone are no error, as in the reference
(`candle-nn/src/var_builder.rs:501-529` reads what it is asked for): they are
returned as a note for the caller to log, unless `strict=True` makes them fatal.

Tensors keep the precision they are stored in: bfloat16 stays bfloat16, a
tensor stored in 32-bit stays 32-bit, half precision is widened to 32-bit
(exact), integer tables become int32.  Conversion to the compute precision is
the business of the part that owns the tensor.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Set, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile, weight_files


@dataclass(frozen=True)
class TensorSpec:
    """What a part expects under a name: the shape, and how random weights fill it."""
    shape: Tuple[int, ...]
    init: str = "matrix"       # "matrix": N(0, 0.02); "norm": 1 + N(0, 0.1); "table": integers
    high: int = 0              # tables: random entries are drawn from 0..high-1 (0: no random fill)


class WeightError(ValueError):
    """Raised once per load, listing everything that is wrong with the checkpoint."""

    def __init__(self, where: str, missing: List[str], unexpected: List[str],
                 wrong_shape: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]],
                 wrong_dtype: List[Tuple[str, str]]):
        self.missing = missing
        self.unexpected = unexpected
        self.wrong_shape = wrong_shape
        self.wrong_dtype = wrong_dtype
        lines = [f"weights in {where} do not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        for name, want, got in wrong_shape:
            lines.append(f"  shape mismatch for {name}: expected {list(want)}, got {list(got)}")
        for name, dt in wrong_dtype:
            lines.append(f"  unsupported dtype for {name}: {dt}")
        super().__init__("\n".join(lines))


_FLOAT = {"F32", "BF16", "F16", "F64"}
_INT = {"I64", "I32", "I16", "I8", "U8"}


def _keep_precision(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return t
    if t.dtype in (torch.float16, torch.float64):
        return t.to(torch.float32)
    if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8):
        if t.numel() and (int(t.max()) > 2**31 - 1 or int(t.min()) < -2**31):
            raise SafetensorsError("integer table does not fit int32")
        return t.to(torch.int32)
    raise SafetensorsError(f"unsupported dtype {t.dtype}")


def load_weights(model_dir: str, expected: Mapping[str, TensorSpec],
                 optional: Iterable[str] = (), strict: bool = False,
                 unused: Optional[List[str]] = None) -> Dict[str, torch.Tensor]:
    """Read every expected tensor from the folder's safetensors files (CPU tensors).

    `optional` names may be absent; when present they are checked like the rest.  Tensors of the
    files that the model does not read are appended to `unused` (when given) and, with `strict`,
    make the load fail.
    """
    optional_set: Set[str] = set(optional)
    files = [SafetensorsFile(p) for p in weight_files(model_dir)]
    try:
        route: Dict[str, SafetensorsFile] = {}
        for f in files:                      # the last file wins on duplicates
            for name in f.entries:
                route[name] = f
        missing = sorted(n for n in expected if n not in route and n not in optional_set)
        unexpected = sorted(n for n in route if n not in expected)
        wrong_shape, wrong_dtype = [], []
        for name, spec in expected.items():
            f = route.get(name)
            if f is None:
                continue
            e = f.entries[name]
            if tuple(e.shape) != tuple(spec.shape):
                wrong_shape.append((name, tuple(spec.shape), tuple(e.shape)))
            if e.dtype not in _FLOAT and not (spec.init == "table" and e.dtype in _INT):
                wrong_dtype.append((name, e.dtype))
        if unused is not None:
            unused.extend(unexpected)
        # (the error names the unexpected tensors too: a misnamed tensor shows up as one missing and one unexpected)
        if missing or wrong_shape or wrong_dtype or (strict and unexpected):
            raise WeightError(model_dir, missing, unexpected, wrong_shape, wrong_dtype)
        out: Dict[str, torch.Tensor] = {}
        for name in expected:
            f = route.get(name)
            if f is not None:
                out[name] = _keep_precision(f.read(name))
        return out
    finally:
        for f in files:
            f.close()
