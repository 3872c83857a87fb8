"""From a `ModelSpec` to the list of tensors it loads (no device needed)."""
from __future__ import annotations

from typing import Dict, Set, Tuple

from ..config.spec import ModelSpec
from ..weights.loader import TensorSpec
from .base import part_class


def layer_tensors(layer) -> Dict[str, TensorSpec]:
    out: Dict[str, TensorSpec] = {}
    for local, ts in part_class("mixer", layer.mixer).tensors(layer.mixer).items():
        out[layer.mixer_prefix + local] = ts
    for local, ts in part_class("ffn", layer.ffn).tensors(layer.ffn).items():
        out[layer.ffn_prefix + local] = ts
    for name, nspec in ((layer.norm_mixer_name, layer.norm_mixer),
                        (layer.norm_ffn_name, layer.norm_ffn)):
        (ts,) = part_class("norm", nspec).tensors(nspec).values()
        out[name] = ts
    return out


def model_tensors(spec: ModelSpec) -> Tuple[Dict[str, TensorSpec], Set[str]]:
    """(every tensor name the model may read -> its spec, the names that may be absent).

    A separate logits head may always be absent: the embedding table then serves, as in the
    reference, which decides by the tensor's presence alone
    (`inferrs-models/src/models/qwen3.rs:369-372`)."""
    expected: Dict[str, TensorSpec] = {
        spec.embed_name: TensorSpec((spec.vocab_size, spec.hidden), "matrix")}
    for layer in spec.layers:
        expected.update(layer_tensors(layer))
    (ts,) = part_class("norm", spec.final_norm).tensors(spec.final_norm).values()
    expected[spec.final_norm_name] = ts
    optional: Set[str] = set()
    if spec.head_name is not None:
        expected[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden), "matrix")
        optional.add(spec.head_name)
    return expected, optional


def generated_tensors(spec: ModelSpec) -> Dict[str, TensorSpec]:
    """What a random model of this spec is made of: everything, the separate logits head only
    when the configuration unties it."""
    expected, _ = model_tensors(spec)
    if spec.head_name is not None and not spec.head_required:
        del expected[spec.head_name]
    return expected
