"""Device arrays behind the cache manager's bookkeeping.

Paged groups: per layer a key array `[pages, n_kv_heads, page_size, head_dim]` and a value array
`[pages, n_kv_heads, head_dim, page_size]` (values are kept transposed inside a page: the
attention kernels multiply probabilities into them along the slots) in the model's precision,
so one page of one head is `page_size * head_dim` contiguous elements.  (The reference keeps `[pages * page_size, n_kv_heads, head_dim]` per layer,
`inferrs-models/src/kv_cache.rs:249-270`, and gathers it into a dense copy per pass; here the
attention kernels read pages through the block table.)  Pages are not cleared on reuse:
attention never reads beyond a request's length.

State layers: one array `[max_seqs, *shape]`; a request's row is cleared when its slot is handed out.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .manager import CacheManager


@dataclass
class LayerCache:
    """What a mixer is handed for its layer.  `writable` is False for a layer that only
    reads the cache of another layer."""
    layer: int
    group: int = -1
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    state: Optional[torch.Tensor] = None
    writable: bool = True

    def reader(self) -> "LayerCache":
        return LayerCache(self.layer, self.group, self.k, self.v, self.state, writable=False)


class CacheStorage:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device):
        self.manager = manager
        self.layers: Dict[int, LayerCache] = {}
        self.arrays = []
        for g in manager.groups:
            need = g.need
            arr = torch.zeros((len(g.layers), 2, max(g.pool.num_pages, 1), need.n_kv_heads,
                               manager.page_size, need.head_dim), dtype=dtype, device=device)
            self.arrays.append(arr)
            for i, layer in enumerate(g.layers):
                self.layers[layer] = LayerCache(
                    layer, g.index, arr[i, 0],
                    arr[i, 1].view(arr.shape[2], need.n_kv_heads, need.head_dim, manager.page_size))
        for st in manager.states:
            arr = torch.zeros((manager.max_seqs, *st.need.shape), dtype=st.need.dtype, device=device)
            self.arrays.append(arr)
            self.layers[st.layer] = LayerCache(st.layer, state=arr)

    def clear_state_slot(self, slot: int) -> None:
        for st in self.manager.states:
            self.layers[st.layer].state[slot].zero_()

    def bytes(self) -> int:
        return sum(a.numel() * a.element_size() for a in self.arrays)
