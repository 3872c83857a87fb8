"""Chat prompts.  The reference picks a template by looking into tokenizer_config.json's
`chat_template` (`inferrs/src/tokenizer.rs:454-470`: a template that mentions "im_start" is ChatML),
with an override per architecture (`tokenizer.rs:323-327`); ChatML is rendered as
`<|im_start|>role\\ncontent<|im_end|>\\n` per message and ends with `<|im_start|>assistant\\n`
(`tokenizer.rs:548-556`).  Here the renderers are a table by name; an architecture's configuration
class may name its default in a `chat_template` attribute, and the folder's tokenizer_config.json
decides where it says something this table knows."""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, List, Optional, Tuple

Messages = List[Tuple[str, str]]       # (role, content)


def _chatml(messages: Messages) -> str:
    return "".join(f"<|im_start|>{role}\n{content}<|im_end|>\n" for role, content in messages) + "<|im_start|>assistant\n"


def _plain(messages: Messages) -> str:
    return "\n".join(content for _role, content in messages)


TEMPLATES: Dict[str, Callable[[Messages], str]] = {"chatml": _chatml, "plain": _plain}


def detect_template(model_dir: str, config=None) -> str:
    """The name of the template for this folder: what tokenizer_config.json's template looks like, else
    the architecture's default, else "plain" (the text as it is)."""
    path = os.path.join(model_dir, "tokenizer_config.json")
    if os.path.isfile(path):
        try:
            with open(path, "r", encoding="utf-8") as f:
                template = json.load(f).get("chat_template")
        except (OSError, ValueError, AttributeError):
            template = None
        if isinstance(template, str) and ("im_start" in template or "im_end" in template):
            return "chatml"
    name = getattr(config, "chat_template", None)
    return name if name in TEMPLATES else "plain"


def render(template: str, user: str, system: Optional[str] = None) -> str:
    messages: Messages = ([("system", system)] if system else []) + [("user", user)]
    return TEMPLATES[template](messages)
