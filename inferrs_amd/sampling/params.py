"""Per-request sampling parameters, with the reference's names, defaults and meanings
(`inferrs/src/sampler.rs:26-130`)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

SAMPLING_EPS = 1e-5          # a temperature below this means greedy (`sampler.rs:114`)


@dataclass
class SamplingParams:
    temperature: float = 0.7          # < 1e-5: greedy
    top_p: float = 0.9                # nucleus; 1.0 disables
    top_k: int = 50                   # 0 disables
    min_p: float = 0.0                # relative to the largest probability; 0 disables
    repetition_penalty: float = 1.1   # 1.0 (or 0.0) disables
    repeat_last_n: int = 64           # tokens of prompt and output the penalties look at; 0 disables them
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    max_tokens: int = 2048            # cap on generated tokens
    seed: Optional[int] = None        # None: a fresh seed per request
    logit_bias: Dict[int, float] = field(default_factory=dict)
    logprobs: bool = False            # report the drawn token's log-probability within the kept list
    top_logprobs: int = 0             # and the first 0..20 entries of that list (needs logprobs)
    extra_stop_token_ids: Tuple[int, ...] = ()
    stop_strings: Tuple[str, ...] = ()  # generation stops when the decoded output ends with one (needs a detokenizer)
    bypass_stop_tokens: bool = False  # run to max_tokens whatever is generated (benchmarks)

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError(f"top_p must lie in (0, 1], got {self.top_p}")
        if self.top_k < 0:
            raise ValueError(f"top_k must be >= 0, got {self.top_k}")
        if not (0.0 <= self.min_p <= 1.0):
            raise ValueError(f"min_p must lie in [0, 1], got {self.min_p}")
        if self.repeat_last_n < 0:
            raise ValueError(f"repeat_last_n must be >= 0, got {self.repeat_last_n}")
        if self.max_tokens < 1:
            raise ValueError(f"max_tokens must be >= 1, got {self.max_tokens}")
        if not (0 <= self.top_logprobs <= 20):
            raise ValueError(f"top_logprobs must lie in 0..20, got {self.top_logprobs}")
        if self.top_logprobs and not self.logprobs:
            raise ValueError("top_logprobs needs logprobs")

    @classmethod
    def greedy(cls, max_tokens: int = 2048, **kw) -> "SamplingParams":
        """Temperature 0 and nothing that reorders logits."""
        return cls(temperature=0.0, top_p=1.0, top_k=0, repetition_penalty=1.0, max_tokens=max_tokens, **kw)

    @property
    def has_penalty(self) -> bool:
        return self.repeat_last_n > 0 and (self.repetition_penalty != 1.0 or self.frequency_penalty != 0.0
                                           or self.presence_penalty != 0.0)

    def draw_temperature(self, n_previous: int) -> float:
        """The temperature that a token after `n_previous` others is drawn at (`sampler.rs:163-179`, `:232-236`):
        the request's own; or 0 for the arg max, which a temperature under `SAMPLING_EPS` means only where nothing
        changes the logits' order (no penalty over a window that holds a token, no bias) and no log-probability is
        asked for; or else `SAMPLING_EPS`, at which the reference draws with the request's random number like at any
        other temperature: among logits that are equal, or closer than a few times 1e-5, after the penalties, every
        one can come."""
        if self.temperature >= SAMPLING_EPS:
            return self.temperature
        untouched = not (self.has_penalty and n_previous > 0) and not self.logit_bias and not self.logprobs
        return 0.0 if untouched else SAMPLING_EPS

    @property
    def is_plain_greedy(self) -> bool:
        """The reference's fast path: arg max of the untouched logits (`sampler.rs:171-179`)."""
        return self.temperature < SAMPLING_EPS and not self.has_penalty and not self.logit_bias and not self.logprobs


@dataclass
class TokenLogprob:
    """What the reference reports for a drawn token (`sampler.rs:119-134`): its log-probability within
    the list that top-k, top-p and min-p kept, and the first `top_logprobs` entries of that list."""
    token_id: int
    logprob: float
    top_logprobs: Tuple[Tuple[int, float], ...] = ()
