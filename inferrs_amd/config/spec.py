"""Architecture-neutral description of a decoder: parts, layers and run order.

A model is data before it is code: a `ModelSpec` lists one `LayerSpec` per
layer, each naming its mixer, feed-forward and norms by `kind` together with
every size and constant they need, and a `schedule` that says in which order
layers run and whose cache each of them uses.  Nothing in here knows a model
family; an architecture is a function from its config.json to a `ModelSpec`
(see `inferrs_amd.config.registry`).

The reference wires the same information into Rust structs per model
(`inferrs-models/src/models/qwen3.rs:28-45`, `:264-290`); here it is explicit
so that layers of one model may differ and parts can be reused.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional, Tuple


class SpecError(ValueError):
    """A specification that the parts or kernels cannot honour."""


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last dimension."""
    size: int
    eps: float
    add_one: bool = False          # weight is stored as (w - 1) when True
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter queries and keys.

    kind "rope": rotate the first `rot_dim` features of each head by
    angle = position * theta**(-2i/rot_dim); pairing "half" pairs feature i
    with i + rot_dim/2, "interleaved" pairs 2i with 2i+1.
    kind "none": nothing is applied.
    `scaling`: None, or a law that changes the angles' frequencies, as (name, factor): ("linear", f)
    divides every frequency by f (positions are read as position / f).  A law that has no entry in
    the position part is refused by name when the part is built.
    """
    kind: str = "rope"
    head_dim: int = 0
    rot_dim: int = 0
    theta: float = 10000.0
    pairing: str = "half"
    scaling: Optional[Tuple[str, float]] = None


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache."""
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: PositionSpec
    qk_norm: Optional[NormSpec] = None     # per-head norm of q and k before rotation
    window: Optional[int] = None           # keys kept: the last `window` positions; None = all
    scale: Optional[float] = None          # None = 1/sqrt(head_dim)
    qkv_bias: bool = False                 # q_proj.bias, k_proj.bias, v_proj.bias are added to the projections
    o_bias: bool = False                   # o_proj.bias is added to the output projection
    kind: str = "attention"

    @property
    def softmax_scale(self) -> float:
        return self.scale if self.scale is not None else self.head_dim ** -0.5


@dataclass(frozen=True)
class GatedMlpSpec:
    """down( act(gate(x)) * up(x) ).  `activation`: "silu", or "gelu_tanh" (GELU in its tanh form); `bias`: every
    projection has a bias vector beside its weight."""
    hidden: int
    intermediate: int
    activation: str = "silu"
    bias: bool = False
    kind: str = "gated_mlp"


@dataclass(frozen=True)
class LayerSpec:
    """One residual block: which parts, how they are arranged, and the tensor names they load from.

    `arrangement` names a registered block class (`parts.register_block`), which says how many
    norms it has and where they stand: "pre_norm" has two, before the mixer and before the
    feed-forward.  `norms[i]` loads its weight from `norm_names[i]`."""
    mixer: Any
    ffn: Any
    norms: Tuple[NormSpec, ...]
    norm_names: Tuple[str, ...]
    mixer_prefix: str
    ffn_prefix: str
    arrangement: str = "pre_norm"


@dataclass(frozen=True)
class EmbeddingSpec:
    """Token ids -> rows of the stream.  kind "embedding": a gather from a [vocab, hidden] table."""
    vocab_size: int
    hidden: int
    name: str
    kind: str = "embedding"


@dataclass(frozen=True)
class HeadSpec:
    """Normed rows -> logits.  kind "lm_head": a product with a [vocab, hidden] matrix stored under
    `name`; when the file has no such tensor (or `name` is None) the embedding table serves.
    `required`: a random model is written with a matrix of its own."""
    vocab_size: int
    hidden: int
    name: Optional[str]
    required: bool = True
    kind: str = "lm_head"


@dataclass(frozen=True)
class ScheduleEntry:
    """One stop in the run order: run `layer` (its weights); its mixer uses a cache.

    By default a stop owns a cache of its own and writes it, so a layer that is named at two
    stops keeps two caches and a request's results do not depend on how its tokens were cut
    into steps.  `cache_of = j` (an earlier stop's index in the schedule) makes this stop
    read stop j's cache and write none.
    """
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: Optional[NormSpec]      # None: the head reads the stream as it is
    final_norm_name: Optional[str]
    embed_name: str
    head_name: Optional[str]            # None: logits use the embedding table
    max_position: int
    head_required: bool = True          # False: use `head_name` if the file has it, else the table
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    embedding: Any = None               # a spec whose `kind` names a registered embedding part; None: EmbeddingSpec
    head: Any = None                    # likewise for the logits head; None: HeadSpec

    def __post_init__(self):
        if self.embedding is None:
            object.__setattr__(self, "embedding", EmbeddingSpec(self.vocab_size, self.hidden, self.embed_name))
        if self.head is None:
            object.__setattr__(self, "head", HeadSpec(self.vocab_size, self.hidden, self.head_name, self.head_required))

    def validate(self) -> None:
        n = len(self.layers)
        if n == 0:
            raise SpecError("a model needs at least one layer")
        if not self.schedule:
            raise SpecError("the schedule is empty")
        if (self.final_norm is None) != (self.final_norm_name is None):
            raise SpecError("a final norm and the name of its weight come together")
        for i, layer in enumerate(self.layers):
            if len(layer.norms) != len(layer.norm_names):
                raise SpecError(f"layer {i}: {len(layer.norms)} norms but {len(layer.norm_names)} names for their weights")
        for i, e in enumerate(self.schedule):
            if not (0 <= e.layer < n):
                raise SpecError(f"schedule stop {i} names layer {e.layer}, outside 0..{n - 1}")
            if e.cache_of is not None:
                if not (0 <= e.cache_of < i):
                    raise SpecError(f"schedule stop {i} reads the cache of stop {e.cache_of}, which is not an earlier stop")
                if self.schedule[e.cache_of].cache_of is not None:
                    raise SpecError(f"schedule stop {i} reads the cache of stop {e.cache_of}, which owns none")

    def cache_stop(self, stop: int) -> int:
        """The schedule stop whose cache stop `stop` uses (itself unless it reads another's)."""
        e = self.schedule[stop]
        return stop if e.cache_of is None else e.cache_of


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    return tuple(ScheduleEntry(i) for i in range(n_layers))
