"""Typed configuration of the Qwen3 dense decoder, read from its config.json keys.

Keys and defaults follow the reference's `to_qwen3_config`
(`inferrs-models/src/config.rs:468-502`): `head_dim` defaults to
`hidden_size / num_attention_heads`, `rms_norm_eps` to 1e-6, `rope_theta` to
1e6, `tie_word_embeddings` to true, `max_position_embeddings` to 40960
(`config.rs:728`).  Unlike the reference, the sizes themselves have no default
here: a config.json without them is an error that names the key.

The reference's model holds no bias, no scaling of the rotation, no window and no
activation but SiLU (`qwen3.rs:28-45`; `hidden_act` is parsed and not used,
`config.rs:291-292`), and it loads a config.json that asks for any of these without
a word, as another model.  Here such a value is an error that names key and value:
`attention_bias` true, a `rope_scaling` that is not null, a `hidden_act` other than
"silu", `use_sliding_window` true, a `layer_types` entry other than "full_attention".
`allow_ignored_keys=True` gives the reference's silence back (the keys are then
ignored as it ignores them).  `sliding_window` and `max_window_layers` alone change
nothing while `use_sliding_window` is false, there and here.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, eos_ids as _eos_ids, opt_number as _opt_number, require_int as _require_int
from .spec import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec,
                   PositionSpec, SpecError, default_schedule)


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    eos_token_ids: Tuple[int, ...] = ()

    architecture = "Qwen3ForCausalLM"
    model_type = "qwen3"
    chat_template = "chatml"        # the family's prompts (`inferrs_amd.chat`), when the folder does not say

    @staticmethod
    def unhonoured_keys(raw: Dict[str, Any]) -> Dict[str, Any]:
        """The keys of `raw` that ask for what this model does not do, with their values."""
        found: Dict[str, Any] = {}
        if raw.get("attention_bias") not in (None, False):
            found["attention_bias"] = raw["attention_bias"]
        if raw.get("rope_scaling") is not None:
            found["rope_scaling"] = raw["rope_scaling"]
        if raw.get("hidden_act") not in (None, "silu"):
            found["hidden_act"] = raw["hidden_act"]
        if raw.get("use_sliding_window") not in (None, False):
            found["use_sliding_window"] = raw["use_sliding_window"]
        types = raw.get("layer_types")
        if types is not None and (not isinstance(types, list) or any(t != "full_attention" for t in types)):
            found["layer_types"] = types
        return found

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], allow_ignored_keys: bool = False) -> "Qwen3Config":
        unhonoured = cls.unhonoured_keys(raw)
        if unhonoured and not allow_ignored_keys:
            what = ", ".join(f"'{k}' = {v!r}" for k, v in unhonoured.items())
            raise ConfigError(
                f"config.json: {what}: {cls.architecture} as built here has no attention bias, no scaled rotation, no "
                "sliding window and no activation but 'silu', and would compute another model's logits "
                "(allow_ignored_keys=True, --allow-ignored-keys on the command line, ignores such keys as the reference does)")
        hidden = _require_int(raw, "hidden_size")
        heads = _require_int(raw, "num_attention_heads")
        kv_heads = raw.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads
        else:
            kv_heads = _require_int(raw, "num_key_value_heads")
        head_dim = raw.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: 'head_dim' is absent and hidden_size {hidden} is not a "
                    f"multiple of num_attention_heads {heads}")
            head_dim = hidden // heads
        else:
            head_dim = _require_int(raw, "head_dim")
        tie = raw.get("tie_word_embeddings")
        if tie is None:
            tie = True
        if not isinstance(tie, bool):
            raise ConfigError(f"config.json: 'tie_word_embeddings' must be a boolean, got {tie!r}")
        eos_ids = _eos_ids(raw)
        maxpos = raw.get("max_position_embeddings")
        maxpos = 40960 if maxpos is None else _require_int(raw, "max_position_embeddings")
        cfg = cls(
            vocab_size=_require_int(raw, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=_require_int(raw, "intermediate_size"),
            num_hidden_layers=_require_int(raw, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=_opt_number(raw, "rms_norm_eps", 1e-6),
            rope_theta=_opt_number(raw, "rope_theta", 1_000_000.0),
            tie_word_embeddings=tie,
            max_position_embeddings=maxpos,
            eos_token_ids=eos_ids,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple "
                f"of num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary pairs")
        if not (self.rms_norm_eps > 0.0):
            raise ConfigError(f"config.json: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not (self.rope_theta > 0.0):
            raise ConfigError(f"config.json: rope_theta must be positive, got {self.rope_theta}")

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        eos = d.pop("eos_token_ids")
        d["architectures"] = [self.architecture]
        d["model_type"] = self.model_type
        d["hidden_act"] = "silu"
        if eos:
            d["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        return d

    def to_spec(self) -> ModelSpec:
        """The layer list of the reference's `Qwen3Model::new` (`qwen3.rs:341-395`)."""
        position = PositionSpec(kind="rope", head_dim=self.head_dim, rot_dim=self.head_dim,
                                theta=self.rope_theta, pairing="half")
        head_norm = NormSpec(size=self.head_dim, eps=self.rms_norm_eps)
        layer_norm = NormSpec(size=self.hidden_size, eps=self.rms_norm_eps)
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            layers.append(LayerSpec(
                mixer=AttentionSpec(hidden=self.hidden_size, n_heads=self.num_attention_heads,
                                    n_kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
                                    position=position, qk_norm=head_norm, window=None),
                ffn=GatedMlpSpec(hidden=self.hidden_size, intermediate=self.intermediate_size,
                                 activation="silu"),
                norms=(layer_norm, layer_norm),
                norm_names=(p + "input_layernorm.weight", p + "post_attention_layernorm.weight"),
                mixer_prefix=p + "self_attn.", ffn_prefix=p + "mlp.", arrangement="pre_norm",
            ))
        spec = ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=self.hidden_size,
            layers=tuple(layers), schedule=default_schedule(self.num_hidden_layers),
            final_norm=layer_norm, final_norm_name="model.norm.weight",
            embed_name="model.embed_tokens.weight", head_name="lm_head.weight",
            head_required=not self.tie_word_embeddings,
            max_position=self.max_position_embeddings, eos_token_ids=self.eos_token_ids)
        spec.validate()
        return spec
