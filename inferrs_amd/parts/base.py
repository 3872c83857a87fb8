"""Interfaces of the parts a layer is made of, and the tables that map a spec's
`kind` to the class that builds it.

A part is built from its spec alone: sizes and constants are parameters, never
the name of a model.  Every part class offers

  * `tensors(spec) -> {local name: TensorSpec}` (a classmethod: no device needed), and
  * `__init__(spec, tensors, dtype, device)` with `tensors` keyed by those local names.

A mixer additionally says what it keeps per request (`cache_need`) and is run
as `forward(ctx, h, cache)`; a feed-forward as `forward(ctx, h)`; a norm as
`forward(x)` or `add_forward(x, delta)` (adds `delta` into `x` in place and
returns the normalised sum); a position encoding as `table(positions)` whose
result the mixer hands to its kernels.

Two optional abilities, for steps of a few rows (decode), where a kernel of its own for "add to
the stream and norm" is all launch and latency: a mixer or feed-forward with `adds_to_stream = True`
finds the stream in `ctx.stream` (and in `ctx.stream_norm` the norm part that reads it next) and may
add its output to it itself, returning `ops.Added` (the new rows' partial sums of squares, and the
rows times that norm's weight) instead of the output; one with `takes_normed_rows = True` may be
handed `ops.NormedRows` instead of normed rows, whose norm its first product finishes (`ops.linear`
and `ops.gated_silu_linear` take them; `.materialize()` gives plain rows).  A norm takes part if it
offers `rows_for_product(x, added)`.  Parts without these attributes are run as ever.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ..weights.loader import TensorSpec


# ---- what a mixer keeps per request ---------------------------------------------------------

@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every cached position, in pages; `window` keeps only the last ones."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class FixedState:
    """State of fixed size per request (shape without the request dimension)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


# ---- registries -----------------------------------------------------------------------------

_TABLES: Dict[str, Dict[str, type]] = {"mixer": {}, "ffn": {}, "norm": {}, "position": {}}


def _register(table: str, kind: str) -> Callable[[type], type]:
    def deco(cls: type) -> type:
        _TABLES[table][kind] = cls
        cls.kind = kind
        return cls
    return deco


def register_mixer(kind: str):
    return _register("mixer", kind)


def register_ffn(kind: str):
    return _register("ffn", kind)


def register_norm(kind: str):
    return _register("norm", kind)


def register_position(kind: str):
    return _register("position", kind)


def part_class(table: str, spec: Any) -> type:
    kind = getattr(spec, "kind", None)
    try:
        return _TABLES[table][kind]
    except KeyError:
        raise KeyError(f"no {table} part is registered for kind {kind!r}; "
                       f"known: {sorted(_TABLES[table])}") from None


# ---- base classes ---------------------------------------------------------------------------

class Part:
    kind = "?"
    # True when `forward` launches the same kernels with the same arguments for every step of
    # one shape, reading everything that changes (positions, pages, slots) from device memory:
    # only then may a decode step that contains the part be captured into a graph and replayed.
    # A part that looks at the host-side lists of the step context must leave this False.
    graph_safe = False

    @classmethod
    def tensors(cls, spec) -> Dict[str, TensorSpec]:
        return {}


class Mixer(Part):
    @classmethod
    def cache_need(cls, spec):
        """`PagedKV`, `FixedState` or None."""
        return None

    def forward(self, ctx, h: torch.Tensor, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def add_forward(self, x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Position(Part):
    def table(self, positions: torch.Tensor):
        """Whatever the mixer's kernels need for these positions (None for no encoding)."""
        return None
