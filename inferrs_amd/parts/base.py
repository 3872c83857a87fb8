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
and `ops.gated_linear` take them; `.materialize()` gives plain rows).  A norm takes part if it
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
    """Keys and values of every cached position, in pages; `window` keeps only the last ones.
    `head_dim` is the width of a key; values have `v_head_dim` (None: the same).  `values=False`:
    one array a layer, the keys' (a mixer that caches a single row a position, a latent one say, from
    which it forms what it needs).  `value_layout`: how a page holds its values: "transposed"
    `[head][dim][slot]`, what this package's attention kernels multiply probabilities into, or
    "rows" `[head][slot][dim]`, as the keys lie."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None
    values: bool = True
    value_layout: str = "transposed"

    def __post_init__(self):
        if self.value_layout not in ("transposed", "rows"):
            raise ValueError(f"PagedKV: value_layout {self.value_layout!r} is neither 'transposed' nor 'rows'")

    @property
    def value_dim(self) -> int:
        if not self.values:
            return 0
        return self.head_dim if self.v_head_dim is None else self.v_head_dim

    def page_elements(self, page_size: int) -> int:
        """Elements that one page of one layer holds (keys and values of all heads)."""
        return self.n_kv_heads * page_size * (self.head_dim + self.value_dim)


@dataclass(frozen=True)
class FixedState:
    """State of fixed size per request (shape without the request dimension)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def bytes_per_request(self) -> int:
        n = 1
        for s in self.shape:
            n *= int(s)
        return n * torch.empty((), dtype=self.dtype).element_size()


# ---- registries -----------------------------------------------------------------------------

_TABLES: Dict[str, Dict[str, type]] = {"mixer": {}, "ffn": {}, "norm": {}, "position": {}, "block": {},
                                       "embedding": {}, "head": {}}


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


def register_block(arrangement: str):
    """A block class: how a layer's mixer, feed-forward and norms are arranged around the stream.
    Looked up by `LayerSpec.arrangement`."""
    return _register("block", arrangement)


def register_embedding(kind: str):
    return _register("embedding", kind)


def register_head(kind: str):
    return _register("head", kind)


def block_class(layer_spec: Any) -> type:
    try:
        return _TABLES["block"][layer_spec.arrangement]
    except KeyError:
        raise KeyError(f"no block is registered for the arrangement {layer_spec.arrangement!r}; "
                       f"known: {sorted(_TABLES['block'])}") from None


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
    # only then may a step that contains the part be captured into a graph and replayed.
    # A part that looks at the host-side lists of the step context must leave this False.
    # A captured decode step may hold several rows of one hidden request (the engine fills a batch
    # up to the size its graph was captured for): the same token at the same position with the same
    # cache slot and state slot, so that every such row writes the same values to the same place.
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


class BlockBase:
    """One layer around the residual stream.  A block class offers

      * `tensors(layer_spec) -> {full tensor name: TensorSpec}` (a classmethod),
      * `__init__(layer_spec, tensors, dtype, device)` with `tensors` keyed by those names,
      * `forward(ctx, x, pending, cache, next_norm) -> (x, pending)`: `x` is the stream, `pending` what the
        block before has left to be added to it (None, a tensor, or `ops.Added` when it is in already), `cache`
        the mixer's `LayerCache`, `next_norm` the `first_norm` of the block that runs next (or the model's
        final norm's stand-in None); the block returns the stream and what IT leaves to be added,
      * `first_norm`: the norm part that reads the stream first in this block, or None (only a block before
        it that prepares rows for exactly this norm looks at it),
      * `parts()`: every part it holds, for the model's questions (may a step be captured, bytes of weights).
    """
    first_norm = None

    @classmethod
    def tensors(cls, layer_spec) -> Dict[str, TensorSpec]:
        raise NotImplementedError

    def parts(self):
        return []

    def forward(self, ctx, x, pending, cache, next_norm=None):
        raise NotImplementedError


class Embedding(Part):
    """Token ids -> the stream's first rows: `forward(ctx) -> [n_tokens, hidden]`; `table` is the
    [vocab, hidden] matrix a tied logits head may share (None if there is none to share)."""
    table = None

    def forward(self, ctx) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Normed rows -> 32-bit logits: `__init__(spec, tensors, dtype, device, embedding)` (the embedding
    part, for a tied head) and `forward(rows) -> float32 [rows, vocab]`."""

    def forward(self, rows: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError
