"""What one step hands to the model: the flattened tokens of all requests in the batch and,
per cache group, where their keys go and where earlier keys lie.

The reference builds the equivalent once per pass for ONE sequence (`PagedPassCache::build`,
`inferrs-models/src/models/attention_utils.rs:252-283`: slot ids for the new tokens, a causal
mask).  Here a step holds any mix of requests, each with a span of new tokens starting at
its cached length, and no mask is built: kernels derive causality from `positions`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch


@dataclass
class GroupStep:
    """Per cache group: `slots[i]` = page * page_size + offset for token i's key and value;
    `block_table[s]` = the pages of request s in logical order."""
    page_size: int
    slots: torch.Tensor          # int32 [n_tokens]
    block_table: torch.Tensor    # int32 [n_seqs, max_pages]


@dataclass
class StepContext:
    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor      # int32 [n_tokens]
    positions: torch.Tensor      # int32 [n_tokens]   absolute position of each token
    token_seq: torch.Tensor      # int32 [n_tokens]   row of the batch each token belongs to
    cu_tokens: torch.Tensor      # int32 [n_seqs + 1] token spans: request s owns cu[s]..cu[s+1]
    state_slots: torch.Tensor    # int32 [n_seqs]     row of the fixed-size state arrays
    want_rows: torch.Tensor      # int32 [n_want]     tokens whose logits are returned
    groups: List[GroupStep]
    # host copies, for launch decisions and for parts that loop on the host
    q_lens: List[int] = field(default_factory=list)
    kv_starts: List[int] = field(default_factory=list)
    state_slots_host: List[int] = field(default_factory=list)
    max_q_len: int = 0
    max_kv_len: int = 0
    _tables: Dict[Any, Any] = field(default_factory=dict)

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1

    def position_table(self, position_part) -> Optional[Any]:
        """The position part's table for this step's tokens, built once per distinct spec."""
        key = position_part.spec
        if key not in self._tables:
            self._tables[key] = position_part.table(self.positions)
        return self._tables[key]
