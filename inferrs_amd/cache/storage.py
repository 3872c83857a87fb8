"""Device arrays behind the cache manager's bookkeeping.

Paged groups: per layer a key array `[pages, n_kv_heads, page_size, head_dim]` and a value array
`[pages, n_kv_heads, value_dim, page_size]` (values are kept transposed inside a page: the
attention kernels multiply probabilities into them along the slots) in the model's precision,
so one page of one head is `page_size * head_dim` contiguous elements.  Keys and values of one
width share one allocation; a mixer whose values are wider or narrower than its keys
(`PagedKV.v_head_dim`) gets two.  A need may ask for its values as rows, `[pages, n_kv_heads,
page_size, value_dim]` (`value_layout="rows"`), or for no value array at all (`values=False`:
`LayerCache.v` is None).  (The reference keeps `[pages * page_size, n_kv_heads, head_dim]` per layer,
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
            pages, ps = max(g.pool.num_pages, 1), manager.page_size
            values = None
            if not need.values:
                keys = torch.zeros((len(g.layers), pages, need.n_kv_heads, ps, need.head_dim), dtype=dtype, device=device)
                self.arrays.append(keys)
            elif need.value_dim == need.head_dim:
                arr = torch.zeros((len(g.layers), 2, pages, need.n_kv_heads, ps, need.head_dim), dtype=dtype, device=device)
                self.arrays.append(arr)
                keys, values = arr[:, 0], arr[:, 1]
            else:
                keys = torch.zeros((len(g.layers), pages, need.n_kv_heads, ps, need.head_dim), dtype=dtype, device=device)
                values = torch.zeros((len(g.layers), pages, need.n_kv_heads, ps, need.value_dim), dtype=dtype, device=device)
                self.arrays += [keys, values]
            for i, layer in enumerate(g.layers):
                v = None
                if values is not None:
                    v = values[i] if need.value_layout == "rows" else values[i].view(pages, need.n_kv_heads, need.value_dim, ps)
                self.layers[layer] = LayerCache(layer, g.index, keys[i], v)
        for st in manager.states:
            arr = torch.zeros((manager.max_seqs, *st.need.shape), dtype=st.need.dtype, device=device)
            self.arrays.append(arr)
            self.layers[st.layer] = LayerCache(st.layer, state=arr)

    def clear_state_slot(self, slot: int) -> None:
        for st in self.manager.states:
            self.layers[st.layer].state[slot].zero_()

    @staticmethod
    def page_bytes(manager: CacheManager, dtype: torch.dtype) -> int:
        """Bytes that one more page in every group costs, over all layers."""
        esize = torch.empty((), dtype=dtype).element_size()
        return sum(len(g.layers) * g.need.page_elements(manager.page_size) * esize for g in manager.groups)

    @staticmethod
    def state_bytes(manager: CacheManager) -> int:
        """Bytes of the fixed-size state arrays: every request slot of every layer that keeps such state."""
        return sum(manager.max_seqs * st.need.bytes_per_request() for st in manager.states)

    def bytes(self) -> int:
        return sum(a.numel() * a.element_size() for a in self.arrays)
