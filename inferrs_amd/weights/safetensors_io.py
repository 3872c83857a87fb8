"""Reader and writer for the safetensors container, written against its layout.

Layout: 8 bytes little-endian header length n, n bytes of JSON mapping each
tensor name to {"dtype", "shape", "data_offsets": [begin, end)} relative to
the byte after the header, then the data.  The reference memory-maps each
file and routes names to files, the last file winning on duplicates
(`candle-core/src/safetensors.rs:423-516`); this module does the same with
`mmap` and `torch.frombuffer`, copying a tensor out only when it is asked for.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Tuple

import numpy as np
import torch

_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int
    end: int


def _numel(shape: Iterable[int]) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


class SafetensorsFile:
    """One memory-mapped file; `entries` lists what it holds."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: truncated file ({size} bytes, no header length)")
        self._f = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen > size - 8:
            raise SafetensorsError(
                f"{path}: truncated file (header says {hlen} bytes, file has {size - 8} after the length)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from e
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header must be a JSON object")
        self.metadata = header.pop("__metadata__", None) or {}
        self.data_start = 8 + hlen
        data_len = size - self.data_start
        self.entries: Dict[str, TensorEntry] = {}
        for name, info in header.items():
            try:
                dtype = info["dtype"]
                shape = tuple(int(s) for s in info["shape"])
                begin, end = (int(x) for x in info["data_offsets"])
            except (KeyError, TypeError, ValueError) as e:
                raise SafetensorsError(f"{path}: malformed header entry for '{name}': {e}") from e
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dtype}")
            want = _numel(shape) * _DTYPES[dtype][1]
            if begin < 0 or end < begin or end - begin != want:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' of shape {list(shape)} and dtype {dtype} needs {want} "
                    f"bytes but its offsets are [{begin}, {end})")
            if end > data_len:
                raise SafetensorsError(
                    f"{path}: truncated file (tensor '{name}' ends at byte {end}, data has {data_len})")
            self.entries[name] = TensorEntry(name, dtype, shape, begin, end)
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor that owns its memory, in the dtype the file stores."""
        e = self.entries[name]
        dtype = _DTYPES[e.dtype][0]
        if e.end == e.begin:
            return torch.empty(e.shape, dtype=dtype)
        raw = np.frombuffer(self._mm, dtype=np.uint8, count=e.end - e.begin,
                            offset=self.data_start + e.begin).copy()
        return torch.from_numpy(raw).view(dtype).reshape(e.shape)

    def close(self) -> None:
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._f.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor],
                      metadata: Optional[Mapping[str, str]] = None) -> None:
    """Write `tensors` (CPU, contiguous or not) in name order."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order: List[str] = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store tensor '{name}' of dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy().data)
    os.replace(tmp, path)


def weight_files(model_dir: str) -> List[str]:
    """`model.safetensors`, else the files of `model.safetensors.index.json`, else all
    `*.safetensors` sorted (`inferrs/src/hub.rs:55-71`, `:523-555`)."""
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            wm = json.load(f).get("weight_map", {})
        files = sorted({os.path.join(model_dir, v) for v in wm.values()})
        if files:
            return files
    files = sorted(os.path.join(model_dir, n) for n in os.listdir(model_dir)
                   if n.endswith(".safetensors"))
    if not files:
        raise SafetensorsError(f"No safetensors files found in {model_dir}")
    return files
