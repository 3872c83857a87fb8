"""One registry from an architecture's name to its configuration class.

The reference detects the architecture by substring match over
`architectures[*]`, then by `model_type`, and bails with
"Unsupported model architecture. architectures=…, model_type=…"
(`inferrs-models/src/config.rs:342-387`).  Here the match is exact and the
table is open: `register_architecture` adds an entry, and an entry is all a
new architecture needs besides parts that may be missing.

An entry is a class with
  * `architecture` and `model_type` strings,
  * `from_dict(raw_config_json) -> config` (validates, names bad keys),
  * `to_dict()` (what the random-weights writer puts into config.json),
  * `to_spec() -> ModelSpec` (layers, run order, tensor names).
"""
from __future__ import annotations

from typing import Any, Dict, Optional, Type

from .base import ConfigError, read_config_json
from .qwen3 import Qwen3Config
from .spec import ModelSpec

_BY_ARCHITECTURE: Dict[str, Type] = {}
_BY_MODEL_TYPE: Dict[str, Type] = {}


def register_architecture(config_cls: Type) -> Type:
    _BY_ARCHITECTURE[config_cls.architecture] = config_cls
    model_type = getattr(config_cls, "model_type", None)
    if model_type:
        _BY_MODEL_TYPE[model_type] = config_cls
    return config_cls


def registered_architectures():
    return sorted(_BY_ARCHITECTURE)


def resolve_architecture(raw: Dict[str, Any]) -> Type:
    archs = raw.get("architectures") or []
    if isinstance(archs, str):
        archs = [archs]
    for a in archs:
        if a in _BY_ARCHITECTURE:
            return _BY_ARCHITECTURE[a]
    model_type: Optional[str] = raw.get("model_type")
    if model_type in _BY_MODEL_TYPE:
        return _BY_MODEL_TYPE[model_type]
    raise ConfigError(
        f"Unsupported model architecture. architectures={archs!r}, model_type={model_type!r}; "
        f"registered: {registered_architectures()}")


def load_config(model_dir: str, allow_ignored_keys: bool = False):
    """config.json of `model_dir` -> typed configuration of its registered architecture.
    `allow_ignored_keys`: handed to the architecture's `from_dict` when set (an architecture that refuses
    values it does not honour then ignores them instead)."""
    raw = read_config_json(model_dir)
    config_cls = resolve_architecture(raw)
    return config_cls.from_dict(raw, allow_ignored_keys=True) if allow_ignored_keys else config_cls.from_dict(raw)


def load_spec(model_dir: str) -> ModelSpec:
    return load_config(model_dir).to_spec()


register_architecture(Qwen3Config)
