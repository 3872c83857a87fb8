"""From a `ModelSpec` to the list of tensors it loads (no device needed)."""
from __future__ import annotations

from typing import Dict, Set, Tuple

from ..config.spec import ModelSpec
from ..weights.loader import TensorSpec
from .base import block_class, part_class


def layer_tensors(layer) -> Dict[str, TensorSpec]:
    return dict(block_class(layer).tensors(layer))


def model_tensors(spec: ModelSpec) -> Tuple[Dict[str, TensorSpec], Set[str]]:
    """(every tensor name the model may read -> its spec, the names that may be absent)."""
    expected: Dict[str, TensorSpec] = dict(part_class("embedding", spec.embedding).tensors(spec.embedding))
    for layer in spec.layers:
        expected.update(layer_tensors(layer))
    if spec.final_norm is not None:
        (ts,) = part_class("norm", spec.final_norm).tensors(spec.final_norm).values()
        expected[spec.final_norm_name] = ts
    head = part_class("head", spec.head)
    expected.update(head.tensors(spec.head))
    optional: Set[str] = set(head.optional(spec.head)) if hasattr(head, "optional") else set()
    return expected, optional


def generated_tensors(spec: ModelSpec) -> Dict[str, TensorSpec]:
    """What a random model of this spec is made of: everything, of the optional tensors those that the
    part asks for (a separate logits head only when the configuration unties it)."""
    expected, optional = model_tensors(spec)
    head = part_class("head", spec.head)
    keep = set(head.generated(spec.head)) if hasattr(head, "generated") else set()
    for name in optional - keep:
        del expected[name]
    return expected
