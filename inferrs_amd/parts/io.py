"""The two ends of a decoder: token ids into the stream (`inferrs-models/src/models/qwen3.rs:398-405`,
a gather without scaling) and normed rows into logits (`qwen3.rs:369-372`, `attention_utils.rs:382-395`:
a product with the head's matrix, or with the embedding table when the file holds no head).  Both are
registered parts, so a model whose ends differ (a scaled embedding, capped logits) brings its own."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import Embedding, Head, register_embedding, register_head
from .linear import Linear, to_compute


@register_embedding("embedding")
class TableEmbedding(Embedding):
    graph_safe = True

    @classmethod
    def tensors(cls, spec) -> Dict[str, TensorSpec]:
        return {spec.name: TensorSpec((spec.vocab_size, spec.hidden), "matrix")}

    def __init__(self, spec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec = spec
        self.table = to_compute(tensors[spec.name], dtype, device)

    def forward(self, ctx) -> torch.Tensor:
        return ops.embed_gather(self.table, ctx.token_ids)


@register_head("lm_head")
class LinearHead(Head):
    graph_safe = True

    @classmethod
    def tensors(cls, spec) -> Dict[str, TensorSpec]:
        if spec.name is None:
            return {}
        return {spec.name: TensorSpec((spec.vocab_size, spec.hidden), "matrix")}

    @classmethod
    def optional(cls, spec):
        """Names that a file may leave out: the embedding table then serves, as in the reference, which
        decides by the tensor's presence alone."""
        return set() if spec.name is None else {spec.name}

    @classmethod
    def generated(cls, spec):
        """Names that a random model is written with."""
        return {spec.name} if spec.name is not None and spec.required else set()

    def __init__(self, spec, tensors: Dict[str, torch.Tensor], dtype, device, embedding=None):
        self.spec = spec
        own = tensors.get(spec.name) if spec.name is not None else None
        if own is not None:
            self.weight = Linear([own], dtype, device).weight
        else:
            table = getattr(embedding, "table", None)
            if table is None or tuple(table.shape) != (spec.vocab_size, spec.hidden):
                raise ValueError("the logits head has no matrix of its own and the embedding offers no table of "
                                 f"[{spec.vocab_size}, {spec.hidden}] to share")
            self.weight = table                      # logits share the embedding table

    def forward(self, rows: torch.Tensor) -> torch.Tensor:
        return ops.linear(rows, self.weight, torch.float32)
