"""What every architecture's configuration shares: the error type, reading config.json, typed
access to its keys, and the stop ids that a model folder declares beside config.json.

Stop ids.  The reference ends a request at the tokenizer's EOS token and at any of a few well-known
end markers that the vocabulary holds (`inferrs/src/tokenizer.rs:337-353`: "<|endoftext|>",
"<|im_end|>", "<end_of_turn>", "<turn|>", "<|end|>").  Here the ids come from, in this order:
`eos_token_id` of config.json, `eos_token_id` of generation_config.json (an integer or a list), the
`eos_token` named by tokenizer_config.json, and those markers, the last two looked up in
tokenizer.json's vocabulary (read as JSON; no tokenizer library is needed for that).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, List, Optional, Sequence, Tuple


class ConfigError(ValueError):
    pass


WELL_KNOWN_STOP_STRINGS = ("<|endoftext|>", "<|im_end|>", "<end_of_turn>", "<turn|>", "<|end|>")


def read_json_object(model_dir: str, name: str, required: bool = True) -> Optional[Dict[str, Any]]:
    path = os.path.join(model_dir, name)
    if not os.path.isfile(path):
        if required:
            raise ConfigError(f"{name} not found in {model_dir}")
        return None
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"Failed to parse {name} in {model_dir}: {e}") from e
    if not isinstance(raw, dict):
        raise ConfigError(f"{name} in {model_dir} must hold a JSON object")
    return raw


def read_config_json(model_dir: str) -> Dict[str, Any]:
    return read_json_object(model_dir, "config.json")


def require_int(raw: Dict[str, Any], key: str, minimum: int = 1) -> int:
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    v = raw[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json: '{key}' must be an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json: '{key}' must be >= {minimum}, got {v}")
    return v


def opt_number(raw: Dict[str, Any], key: str, default: float) -> float:
    v = raw.get(key)
    if v is None:
        return float(default)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: '{key}' must be a number, got {v!r}")
    return float(v)


def eos_ids(raw: Dict[str, Any], where: str = "config.json") -> Tuple[int, ...]:
    """`eos_token_id`: absent, an integer, or a list of integers."""
    eos = raw.get("eos_token_id")
    if eos is None:
        return ()
    if isinstance(eos, int) and not isinstance(eos, bool):
        return (eos,)
    if isinstance(eos, list) and all(isinstance(e, int) and not isinstance(e, bool) for e in eos):
        return tuple(eos)
    raise ConfigError(f"{where}: 'eos_token_id' must be an integer or a list, got {eos!r}")


def _vocabulary_ids(tokenizer_json: Dict[str, Any], strings: Sequence[str]) -> Dict[str, int]:
    found: Dict[str, int] = {}
    model = tokenizer_json.get("model")
    vocab = model.get("vocab") if isinstance(model, dict) else None
    if isinstance(vocab, dict):
        for s in strings:
            if isinstance(vocab.get(s), int):
                found[s] = vocab[s]
    added = tokenizer_json.get("added_tokens")
    if isinstance(added, list):
        for entry in added:
            if isinstance(entry, dict) and entry.get("content") in strings and isinstance(entry.get("id"), int):
                found[entry["content"]] = entry["id"]
    return found


def folder_stop_ids(model_dir: str, config_ids: Sequence[int] = ()) -> Tuple[int, ...]:
    """Every token id that ends a request of this folder's model, without repeats, config.json's first."""
    ids: List[int] = [int(i) for i in config_ids]

    def add(i: int) -> None:
        if i not in ids:
            ids.append(i)

    generation = read_json_object(model_dir, "generation_config.json", required=False)
    if generation is not None:
        for i in eos_ids(generation, "generation_config.json"):
            add(i)
    tokenizer = read_json_object(model_dir, "tokenizer.json", required=False)
    if tokenizer is not None:
        wanted = list(WELL_KNOWN_STOP_STRINGS)
        tok_config = read_json_object(model_dir, "tokenizer_config.json", required=False)
        eos_token = tok_config.get("eos_token") if tok_config is not None else None
        if isinstance(eos_token, dict):                    # {"content": "..."} in some folders
            eos_token = eos_token.get("content")
        if isinstance(eos_token, str):
            wanted.insert(0, eos_token)
        found = _vocabulary_ids(tokenizer, wanted)
        for s in wanted:
            if s in found:
                add(found[s])
    return tuple(ids)
