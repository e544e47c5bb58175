"""Device memory behind the cache manager's page ids and state slots.

Each layer that owns a cache has its keys and values as two tensors
`[pages, kv_heads, page_size, head_dim]` in the path's dtype (bfloat16 for
serving, float32 on the 32-bit path; the reference's widest row type is F16,
include/liyab/types.h:208-213). Layers of one group share page ids, so one
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
    """What a mixer gets for its layer: the group it belongs to and its memory."""

    group: int
    k: torch.Tensor
    v: torch.Tensor


class CacheStorage:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device, state_specs: Dict[int, StateSpec] | None = None):
        self.manager = manager
        self.dtype = dtype
        self.device = torch.device(device)
        self.layers: Dict[int, LayerCache] = {}
        for g in manager.groups:
            shape = (g.pool.num_pages, g.spec.n_kv_head, manager.page_size, g.spec.head_dim)
            for layer in g.layers:
                self.layers[layer] = LayerCache(
                    group=g.index,
                    k=torch.empty(shape, dtype=dtype, device=self.device),
                    v=torch.empty(shape, dtype=dtype, device=self.device),
                )
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
            n += 2 * len(g.layers) * g.spec.n_kv_head * g.spec.head_dim * self.dtype.itemsize
        return n

    def bytes_allocated(self) -> int:
        return sum(c.k.numel() * c.k.element_size() * 2 for c in self.layers.values()) + sum(
            t.numel() * t.element_size() for t in self.states.values())
