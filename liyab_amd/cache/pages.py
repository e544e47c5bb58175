"""The cache manager: pages of keys and values, block tables, state slots.

The bookkeeping itself is native (`csrc/host/cache_manager.{h,cpp}`, where the rules and
their sources in the reference are written down); this module is its Python face: it maps
the callers' request ids to the state slots the native side knows requests by, turns
status codes into exceptions, and describes the groups of layers. One pool per group is
shared by every live request, so pages a finished request gives back are used again by
the next; a request that cannot get its pages changes nothing (`OutOfPages`).

Beside the pages, each request holds one slot of fixed-size state for mixers that keep
state instead of keys (the reference's `Context::states_`, src/core/transformer.h:853-865,
1296-1303); a model without such mixers has slots of zero bytes.

This is bookkeeping on the host only; the device memory that page ids and slots index
lives in `CacheStorage`.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, Hashable, List, Sequence, Tuple

import numpy as np

from .. import host
from ..errors import InvalidArgument

UNMAPPED = -1
_I32P = ctypes.POINTER(ctypes.c_int32)
_IP = ctypes.POINTER(ctypes.c_int)


def _ints(values) -> np.ndarray:
    return np.ascontiguousarray(values, dtype=np.intc)


def _ip(a: np.ndarray):
    return a.ctypes.data_as(_IP)


@dataclass(frozen=True)
class KVSpec:
    """What a mixer that keeps rows per position needs of the cache: pages of `rows`, each a
    named plane `(name, heads, width)` stored as [pages, heads, page_size, width]. Attention keeps
    keys and values of one shape, which is what `rows` is when it is left empty: ("k", n_kv_head,
    head_dim) and ("v", n_kv_head, head_dim). A mixer with rows of other widths, or with one
    compressed row a position instead of a key and a value, names its own planes (the reference
    pads every layer's rows to its widest instead, src/core/transformer.cpp:2875-2890)."""

    n_kv_head: int
    head_dim: int
    window: int = 0  # 0: every position is kept; W > 0: only the last W are read
    rows: Tuple[Tuple[str, int, int], ...] = ()

    @property
    def planes(self) -> Tuple[Tuple[str, int, int], ...]:
        return self.rows or (("k", self.n_kv_head, self.head_dim), ("v", self.n_kv_head, self.head_dim))

    @property
    def key(self) -> tuple:
        """Layers with equal keys share a group: the same pages, one block table a request."""
        return (self.planes, self.window)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state of a mixer: a tensor of `shape` per slot."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


class PagePool:
    """Page ids 0..n-1 with a free stack; a page is held by at most one owner. (A pool on its
    own; a manager's pools are reached through `CacheManager.groups[i].pool`.)"""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise InvalidArgument("a page pool needs at least one page")
        self.num_pages = num_pages
        self._lib = host.lib()
        self._h = self._lib.liyab_pool_create(num_pages)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.liyab_pool_destroy(self._h)
            self._h = None

    @property
    def free_pages(self) -> int:
        return self._lib.liyab_pool_free_pages(self._h)

    @property
    def pages_in_use(self) -> int:
        return self.num_pages - self.free_pages

    @property
    def peak_in_use(self) -> int:
        return self._lib.liyab_pool_peak(self._h)

    def allocate(self, n: int) -> List[int]:
        out = np.empty(max(n, 1), dtype=np.int32)
        host.check(self._lib.liyab_pool_allocate(self._h, n, out.ctypes.data_as(_I32P)))
        return out[:n].tolist()

    def release(self, pages: Sequence[int]) -> None:
        a = np.ascontiguousarray(pages, dtype=np.int32)
        host.check(self._lib.liyab_pool_release(self._h, a.ctypes.data_as(_I32P), len(a)))

    def check(self) -> None:
        host.check(self._lib.liyab_pool_check(self._h))


class _GroupPool:
    """The counters of one of a manager's pools."""

    def __init__(self, manager: "CacheManager", group: int, num_pages: int):
        self._m, self._g, self.num_pages = manager, group, num_pages

    @property
    def free_pages(self) -> int:
        return self._m._lib.liyab_cm_free_pages(self._m._h, self._g)

    @property
    def pages_in_use(self) -> int:
        return self.num_pages - self.free_pages

    @property
    def peak_in_use(self) -> int:
        return self._m._lib.liyab_cm_peak_in_use(self._m._h, self._g)


@dataclass
class CacheGroup:
    """Layers with the same needs; they share page ids, each has its own memory."""

    index: int
    spec: KVSpec
    layers: List[int]
    pool: _GroupPool


class CacheManager:
    def __init__(self, group_specs: Sequence[Tuple[KVSpec, Sequence[int]]], *, page_size: int,
                 num_pages: int | Sequence[int], max_requests: int, max_positions: int):
        """`group_specs`: (spec, layers) per group. `num_pages`: one number for
        every group or one per group. `max_positions`: the longest context a
        request may reach (the model's or the user's limit)."""
        if page_size <= 0:
            raise InvalidArgument("page_size must be positive")
        if max_requests <= 0:
            raise InvalidArgument("max_requests must be positive")
        if max_positions <= 0:
            raise InvalidArgument("max_positions must be positive")
        self.page_size = page_size
        self.max_positions = max_positions
        self.max_requests = max_requests
        counts = [num_pages] * len(group_specs) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(group_specs):
            raise InvalidArgument("one page count per group is needed")
        if any(n <= 0 for n in counts):
            raise InvalidArgument("a page pool needs at least one page")
        if len(group_specs) > host.MAX_GROUPS:
            raise InvalidArgument(f"{len(group_specs)} cache groups; at most {host.MAX_GROUPS} are taken")
        self._lib = host.lib()
        windows = _ints([spec.window for spec, _ in group_specs])
        self._h = self._lib.liyab_cm_create(len(group_specs), _ip(windows), _ip(_ints(counts)), page_size, max_requests,
                                            max_positions)
        if not self._h:
            raise InvalidArgument(self._lib.liyab_host_last_error().decode())
        self.groups = [CacheGroup(i, spec, list(layers), _GroupPool(self, i, n))
                       for i, ((spec, layers), n) in enumerate(zip(group_specs, counts))]
        self.group_of_layer: Dict[int, int] = {l: g.index for g in self.groups for l in g.layers}
        self.max_blocks = self._lib.liyab_cm_max_blocks(self._h)
        self._slots: Dict[Hashable, int] = {}
        # the native tables, a row per state slot (the memory never moves)
        self._table_rows = [np.ctypeslib.as_array(self._lib.liyab_cm_table_rows(self._h, g),
                                                  shape=(max_requests, self.max_blocks)) for g in range(len(self.groups))]
        self._need = np.zeros(max(len(self.groups), 1), dtype=np.intc)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.liyab_cm_destroy(self._h)
            self._h = None

    @property
    def handle(self):
        """The native manager, for the native calls that take one (a step's metadata)."""
        return self._h

    # -- requests -----------------------------------------------------------
    def open(self, rid: Hashable) -> int:
        """Registers a request and gives it a state slot; returns the slot."""
        if rid in self._slots:
            raise InvalidArgument(f"request {rid!r} is already open")
        slot = ctypes.c_int(-1)
        host.check(self._lib.liyab_cm_open(self._h, ctypes.byref(slot)))
        self._slots[rid] = slot.value
        return slot.value

    def bind(self, rid: Hashable, slot: int) -> None:
        """The native scheduler opened `slot` for `rid` (it works on the native manager itself)."""
        self._slots[rid] = slot

    def unbind(self, rid: Hashable) -> None:
        """The native scheduler closed the request's slot."""
        self._slots.pop(rid, None)

    def is_open(self, rid: Hashable) -> bool:
        return rid in self._slots

    def close(self, rid: Hashable) -> None:
        """Gives back everything the request holds."""
        host.check(self._lib.liyab_cm_close(self._h, self._slots.pop(rid)))

    def length(self, rid: Hashable) -> int:
        return self._lib.liyab_cm_length(self._h, self._slots[rid])

    def slot(self, rid: Hashable) -> int:
        return self._slots[rid]

    def live_requests(self) -> List[Hashable]:
        return list(self._slots)

    # -- pages --------------------------------------------------------------
    def _pages_for(self, n_positions: int) -> int:
        return -(-n_positions // self.page_size)

    def pages_needed(self, rid: Hashable, new_length: int) -> List[int]:
        """New pages per group that `reserve(rid, new_length)` would take."""
        self._lib.liyab_cm_pages_needed(self._h, self._slots[rid], new_length, _ip(self._need))
        return self._need[:len(self.groups)].tolist()

    def can_reserve(self, wants: Sequence[Tuple[Hashable, int]], new_lengths: Sequence[int] = ()) -> bool:
        """Whether `reserve(wants)` would succeed, with requests that are not
        open yet and would come to hold `new_lengths` positions counted in."""
        need = [0] * len(self.groups)
        for rid, new_length in wants:
            for gi, n in enumerate(self.pages_needed(rid, new_length)):
                need[gi] += n
        for length in new_lengths:
            for gi in range(len(self.groups)):
                need[gi] += self._pages_for(length)
        return all(n <= g.pool.free_pages for n, g in zip(need, self.groups))

    def free_slots(self) -> int:
        return self._lib.liyab_cm_free_slots(self._h)

    def reserve(self, wants: Sequence[Tuple[Hashable, int]]) -> None:
        """Maps pages so that each request can hold `new_length` positions.
        All or nothing: raises OutOfPages (or ContextFull) before anything
        changed."""
        slots = _ints([self._slots[rid] for rid, _ in wants])
        lengths = _ints([n for _, n in wants])
        host.check(self._lib.liyab_cm_reserve(self._h, _ip(slots), _ip(lengths), len(slots)))

    def reserve_more(self, slots: np.ndarray, extra: np.ndarray) -> np.ndarray:
        """`reserve` for requests named by slot that each bring `extra[i]` more positions than
        they hold (intc arrays); returns the lengths they will have."""
        out = np.empty(len(slots), dtype=np.intc)
        host.check(self._lib.liyab_cm_reserve_more(self._h, _ip(slots), _ip(extra), len(slots), _ip(out)))
        return out

    def commit(self, rid: Hashable, new_length: int) -> None:
        """The request now holds `new_length` positions. Windowed groups give
        back the pages no later query can see: a query at position p >= length
        reads [p - W + 1, p], so pages wholly below length - W + 1 go."""
        host.check(self._lib.liyab_cm_commit(self._h, self._slots[rid], new_length))

    def commit_slots(self, slots: np.ndarray, new_lengths: np.ndarray) -> None:
        """`commit` for several requests named by slot (intc arrays), in one call."""
        host.check(self._lib.liyab_cm_commit_many(self._h, _ip(slots), _ip(new_lengths), len(slots)))

    def truncate(self, rid: Hashable, length: int) -> None:
        """Forgets positions >= length; pages wholly past it are given back
        (the reference's truncate, kv_cache.cpp:418-439). A windowed group
        cannot go back below what it has already released."""
        host.check(self._lib.liyab_cm_truncate(self._h, self._slots[rid], length))

    def block_table(self, rid: Hashable, group: int = 0) -> List[int]:
        slot = self._slots[rid]
        n = self._lib.liyab_cm_table_length(self._h, slot, group)
        return self._table_rows[group][slot, :n].tolist()

    def table_rows(self, group: int = 0) -> np.ndarray:
        """int32 [max_requests, max_blocks]: the block table of the request in each state slot
        (UNMAPPED where nothing is mapped). Read-only for callers."""
        return self._table_rows[group]

    def slot_of_position(self, rid: Hashable, group: int, position: int) -> int:
        """page * page_size + offset for a mapped position."""
        table = self.block_table(rid, group)
        lp = position // self.page_size
        if lp >= len(table) or table[lp] == UNMAPPED:
            raise InvalidArgument(f"position {position} of request {rid!r} is not mapped in group {group}")
        return table[lp] * self.page_size + position % self.page_size

    # -- accounting -----------------------------------------------------------
    def pages_in_use(self, group: int = 0) -> int:
        return self.groups[group].pool.pages_in_use

    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.free_pages

    def check(self) -> None:
        """Invariants over pools, tables and slots (used by the tests)."""
        host.check(self._lib.liyab_cm_check(self._h))
        slots = list(self._slots.values())
        assert len(set(slots)) == len(slots), "a state slot is held twice"
        assert len(slots) + self.free_slots() == self.max_requests, "a state slot was lost"
