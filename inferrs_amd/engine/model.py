"""A decoder assembled from a `ModelSpec`: embedding, the blocks in schedule order, final norm
and logits at the wanted rows (`inferrs-models/src/models/qwen3.rs:398-440`,
`attention_utils.rs:382-395`).  Nothing here names an architecture."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import ModelSpec
from ..parts.base import block_class, part_class
from ..parts.linear import Linear
from .batch import StepContext

DTYPES = {"float32": torch.float32, "f32": torch.float32, "fp32": torch.float32,
          "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine computes in float32 or bfloat16, not {name}")
        return name
    try:
        return DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}; choose bfloat16 or float32") from None


class DecoderModel:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device):
        """`tensors`: every tensor of `model_tensors(spec)` by name, in its stored precision,
        on any device.  Entries are dropped from the dict as they are taken over."""
        spec.validate()
        self.spec, self.dtype, self.device = spec, dtype, torch.device(device)

        def take(names) -> Dict[str, torch.Tensor]:
            return {n: tensors.pop(n) for n in list(names) if n in tensors}

        embedding_cls = part_class("embedding", spec.embedding)
        self.embedding = embedding_cls(spec.embedding, take(embedding_cls.tensors(spec.embedding)), dtype, device)
        head_cls = part_class("head", spec.head)
        self.head = head_cls(spec.head, take(head_cls.tensors(spec.head)), dtype, device, embedding=self.embedding)
        self.blocks = []
        for layer in spec.layers:
            cls = block_class(layer)
            self.blocks.append(cls(layer, take(cls.tensors(layer)), dtype, device))
        self.final_norm = None
        if spec.final_norm is not None:
            self.final_norm = part_class("norm", spec.final_norm)(
                spec.final_norm, {"weight": tensors.pop(spec.final_norm_name)}, dtype, device)

    @property
    def graph_safe(self) -> bool:
        """Whether every part allows a decode step to be captured and replayed."""
        parts = [self.embedding, self.head, self.final_norm]
        for b in self.blocks:
            parts += list(b.parts())
        return all(getattr(p, "graph_safe", False) for p in parts if p is not None)

    def all_parts(self):
        parts = [self.embedding, self.head, self.final_norm]
        for b in self.blocks:
            parts += list(b.parts())
        return [p for p in parts if p is not None]

    def load_notes(self, page_size: int):
        """What the parts have to say once about how they will run (a part may offer `load_notes(page_size)`):
        every different note once, in the order of the parts."""
        notes = []
        for p in self.all_parts():
            for note in (p.load_notes(page_size) if hasattr(p, "load_notes") else []):
                if note not in notes:
                    notes.append(note)
        return notes

    def cache_needs(self) -> Dict[int, object]:
        """Schedule stop that owns a cache -> what its mixer keeps per request."""
        needs: Dict[int, object] = {}
        for stop, e in enumerate(self.spec.schedule):
            if e.cache_of is None:
                mixer = self.spec.layers[e.layer].mixer
                needs[stop] = part_class("mixer", mixer).cache_need(mixer)
        return needs

    def forward(self, ctx: StepContext, storage) -> torch.Tensor:
        """Runs the step's tokens through every stop of the schedule (which appends to the
        caches) and returns float32 logits `[n_want, vocab]`."""
        x = self.embedding.forward(ctx)
        pending = None                               # a block's output that is not added to x yet
        for stop, e in enumerate(self.spec.schedule):
            cache = storage.layers.get(self.spec.cache_stop(stop))
            if cache is not None and e.cache_of is not None:
                cache = cache.reader()
            after = self.spec.schedule[stop + 1].layer if stop + 1 < len(self.spec.schedule) else None
            next_norm = self.blocks[after].first_norm if after is not None else None
            x, pending = self.blocks[e.layer].forward(ctx, x, pending, cache, next_norm)
        n_want = ctx.want_rows.numel()
        if n_want == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        if isinstance(pending, ops.Partials):        # the last product is still split along k
            pending = pending.materialize()
        xs = ops.gather_rows(x, ctx.want_rows)
        added = pending is None or isinstance(pending, ops.Added)   # the last block has left nothing to add
        if self.final_norm is None:
            h = xs if added else ops.add_inplace(xs, ops.gather_rows(pending, ctx.want_rows))
        elif added:
            h = self.final_norm.forward(xs)
        else:
            h = self.final_norm.add_forward(xs, ops.gather_rows(pending, ctx.want_rows))
        return self.head.forward(h)

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        def add(t):
            nonlocal total
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr()); total += t.numel() * t.element_size()
        parts = [self.embedding, self.head, self.final_norm]
        for b in self.blocks:
            parts += list(b.parts())
        for part in parts:
            if part is None:
                continue
            for v in vars(part).values():
                if isinstance(v, torch.Tensor):
                    add(v)
                elif isinstance(v, Linear):
                    add(v.weight)
                    add(v.bias)
        return total
