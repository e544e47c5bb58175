"""Device memory behind the cache manager's page ids and state slots.

Each layer that owns a cache has one tensor `[pages, heads, page_size, width]`
for each plane of rows its mixer's `KVSpec` names (attention: keys and values,
two tensors `[pages, kv_heads, page_size, head_dim]`) in the path's dtype
(bfloat16 for serving, float32 on the 32-bit path; the reference's widest row
type is F16, include/liyab/types.h:208-213). Layers of one group share page ids, so one
block table per request and group addresses all of them, as one pool page
holds every layer of a unit in the reference (src/core/kv_cache.cpp:305-320).
Pages are not cleared: kernels read only positions below a request's length.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .pages import CacheManager, StateSpec

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


@dataclass
class LayerCache:
    """What a mixer gets for its layer: the group it belongs to and its memory, a tensor
    [pages, heads, page_size, width] for each plane of rows its `KVSpec` names."""

    group: int
    rows: Dict[str, torch.Tensor]

    @property
    def k(self) -> torch.Tensor:
        return self.rows["k"]

    @property
    def v(self) -> torch.Tensor:
        return self.rows["v"]


class CacheStorage:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device, state_specs: Dict[int, StateSpec] | None = None):
        self.manager = manager
        self.dtype = dtype
        self.device = torch.device(device)
        self.layers: Dict[int, LayerCache] = {}
        for g in manager.groups:
            for layer in g.layers:
                self.layers[layer] = LayerCache(group=g.index, rows={
                    name: torch.empty((g.pool.num_pages, heads, manager.page_size, width), dtype=dtype, device=self.device)
                    for name, heads, width in g.spec.planes})
        self.states: Dict[int, torch.Tensor] = {}
        for layer, spec in (state_specs or {}).items():
            self.states[layer] = torch.zeros((manager.max_requests, *spec.shape), dtype=_DTYPES[spec.dtype],
                                             device=self.device)

    def layer(self, index: int) -> Optional[LayerCache]:
        return self.layers.get(index)

    def state(self, index: int) -> Optional[torch.Tensor]:
        return self.states.get(index)

    def reset_slot(self, slot: int) -> None:
        """A slot starts at zero for each new request."""
        from ..kernels import ops

        for t in self.states.values():
            ops.fill_(t[slot], 0)

    def bytes_per_token(self) -> int:
        n = 0
        for g in self.manager.groups:
            n += len(g.layers) * sum(heads * width for _, heads, width in g.spec.planes) * self.dtype.itemsize
        return n

    def bytes_allocated(self) -> int:
        return sum(t.numel() * t.element_size() for c in self.layers.values() for t in c.rows.values()) + sum(
            t.numel() * t.element_size() for t in self.states.values())
