"""A plain cache manager in Python: the reference the native one (liyab_amd/csrc/host/) is
compared with, operation by operation, in tests/test_cache.py. Same rules as the native one:
pages of `page_size` positions mapped on demand (the reference's reserve,
src/core/kv_cache.cpp:249-265), a table per request and group (include/liyab/kv_cache.h:358-365),
windowed groups that give back the pages a window has passed (kv_cache.cpp:474-487), truncate
(kv_cache.cpp:418-439), one free stack per pool (the most recently freed page is used first).
It shares no code with the product."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from liyab_amd.errors import Busy, ContextFull, InvalidArgument, OutOfPages

UNMAPPED = -1


@dataclass(frozen=True)
class KVSpec:
    """What an attention-like mixer needs of the cache."""

    n_kv_head: int
    head_dim: int
    window: int = 0  # 0: every position is kept; W > 0: only the last W are read

    @property
    def key(self) -> Tuple[int, int, int]:
        return (self.n_kv_head, self.head_dim, self.window)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state of a mixer: a tensor of `shape` per slot."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


class PagePool:
    """Page ids 0..n-1 with a free stack; a page is held by at most one owner."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise InvalidArgument("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # pop() gives page 0 first
        self._held = [False] * num_pages
        self.peak_in_use = 0

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def pages_in_use(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self, n: int) -> List[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} free of {self.num_pages}")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            assert not self._held[p], f"page {p} handed out twice"
            self._held[p] = True
        self.peak_in_use = max(self.peak_in_use, self.pages_in_use)
        return out

    def release(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not (0 <= p < self.num_pages) or not self._held[p]:
                raise AssertionError(f"page {p} freed but not held")
            self._held[p] = False
            self._free.append(p)  # most recently freed is used first

    def check(self) -> None:
        """Invariants: every page is free or held, none both, none twice."""
        assert len(set(self._free)) == len(self._free), "a page is on the free list twice"
        for p in self._free:
            assert not self._held[p], f"page {p} is free and held"
        assert sum(self._held) + len(self._free) == self.num_pages, "a page was lost"


@dataclass
class CacheGroup:
    """Layers with the same needs; they share page ids, each has its own memory."""

    index: int
    spec: KVSpec
    layers: List[int]
    pool: PagePool


@dataclass
class _Request:
    length: int = 0  # positions committed
    reserved: int = 0  # positions whose pages are mapped (>= length)
    tables: List[List[int]] = field(default_factory=list)  # per group: logical page -> pool page
    first_kept: List[int] = field(default_factory=list)  # per group: first logical page still mapped
    slot: int = UNMAPPED


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
        self.page_size = page_size
        self.max_positions = max_positions
        self.max_requests = max_requests
        counts = [num_pages] * len(group_specs) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(group_specs):
            raise InvalidArgument("one page count per group is needed")
        self.groups = [CacheGroup(i, spec, list(layers), PagePool(n))
                       for i, ((spec, layers), n) in enumerate(zip(group_specs, counts))]
        self.group_of_layer: Dict[int, int] = {l: g.index for g in self.groups for l in g.layers}
        self._requests: Dict[Hashable, _Request] = {}
        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        self.max_blocks = max(1, -(-max_positions // page_size))
        # the same tables as arrays, a row per state slot: the step function gathers a batch's rows at once
        self._table_rows = [np.full((max_requests, self.max_blocks), UNMAPPED, dtype=np.int32) for _ in self.groups]

    # -- requests -----------------------------------------------------------
    def open(self, rid: Hashable) -> int:
        """Registers a request and gives it a state slot; returns the slot."""
        if rid in self._requests:
            raise InvalidArgument(f"request {rid!r} is already open")
        if not self._free_slots:
            raise Busy(f"all {self.max_requests} request slots are in use")
        r = _Request(tables=[[] for _ in self.groups], first_kept=[0 for _ in self.groups],
                     slot=self._free_slots.pop())
        self._requests[rid] = r
        return r.slot

    def is_open(self, rid: Hashable) -> bool:
        return rid in self._requests

    def close(self, rid: Hashable) -> None:
        """Gives back everything the request holds."""
        r = self._requests.pop(rid)
        for g, table, rows in zip(self.groups, r.tables, self._table_rows):
            g.pool.release([p for p in table if p != UNMAPPED])
            rows[r.slot, :] = UNMAPPED
        self._free_slots.append(r.slot)

    def length(self, rid: Hashable) -> int:
        return self._requests[rid].length

    def slot(self, rid: Hashable) -> int:
        return self._requests[rid].slot

    def live_requests(self) -> List[Hashable]:
        return list(self._requests)

    # -- pages --------------------------------------------------------------
    def _pages_for(self, n_positions: int) -> int:
        return -(-n_positions // self.page_size)

    def pages_needed(self, rid: Hashable, new_length: int) -> List[int]:
        """New pages per group that `reserve(rid, new_length)` would take."""
        r = self._requests[rid]
        return [max(0, self._pages_for(new_length) - len(t)) for t in r.tables]

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
        return len(self._free_slots)

    def reserve(self, wants: Sequence[Tuple[Hashable, int]]) -> None:
        """Maps pages so that each request can hold `new_length` positions.
        All or nothing: raises OutOfPages (or ContextFull) before anything
        changed."""
        need = [0] * len(self.groups)
        for rid, new_length in wants:
            r = self._requests[rid]
            if new_length > self.max_positions:
                raise ContextFull(f"request {rid!r} would reach {new_length} positions; the context holds {self.max_positions}")
            if new_length < r.length:
                raise InvalidArgument("reserve cannot shrink a request; use truncate")
            for gi, n in enumerate(self.pages_needed(rid, new_length)):
                need[gi] += n
        for n, g in zip(need, self.groups):
            if n > g.pool.free_pages:
                raise OutOfPages(f"group {g.index}: {n} pages wanted, {g.pool.free_pages} free of {g.pool.num_pages}")
        for rid, new_length in wants:
            r = self._requests[rid]
            for g, table, rows in zip(self.groups, r.tables, self._table_rows):
                new = g.pool.allocate(max(0, self._pages_for(new_length) - len(table)))
                if new:
                    rows[r.slot, len(table):len(table) + len(new)] = new
                    table.extend(new)
            r.reserved = max(r.reserved, new_length)

    def commit(self, rid: Hashable, new_length: int) -> None:
        """The request now holds `new_length` positions. Windowed groups give
        back the pages no later query can see: a query at position p >= length
        reads [p - W + 1, p], so pages wholly below length - W + 1 go."""
        r = self._requests[rid]
        if self.groups and new_length > len(r.tables[0]) * self.page_size:
            raise InvalidArgument("commit past the reserved pages")
        r.length = new_length
        for gi, g in enumerate(self.groups):
            if g.spec.window <= 0:
                continue
            first_needed = max(0, new_length - g.spec.window + 1)
            keep_from = first_needed // self.page_size
            table = r.tables[gi]
            gone = []
            for lp in range(r.first_kept[gi], min(keep_from, len(table))):
                if table[lp] != UNMAPPED:
                    gone.append(table[lp])
                    table[lp] = UNMAPPED
                    self._table_rows[gi][r.slot, lp] = UNMAPPED
            r.first_kept[gi] = max(r.first_kept[gi], min(keep_from, len(table)))
            g.pool.release(gone)

    def truncate(self, rid: Hashable, length: int) -> None:
        """Forgets positions >= length; pages wholly past it are given back
        (the reference's truncate, kv_cache.cpp:418-439). A windowed group
        cannot go back below what it has already released."""
        r = self._requests[rid]
        if length > r.length:
            raise InvalidArgument("truncate cannot grow a request")
        keep = self._pages_for(length)
        for gi, g in enumerate(self.groups):  # refusals first: a truncate that fails changes nothing
            if g.spec.window > 0 and r.first_kept[gi] * self.page_size > max(0, length - g.spec.window + 1):
                raise InvalidArgument("a windowed group has already released what this truncate needs")
        for gi, g in enumerate(self.groups):
            table = r.tables[gi]
            g.pool.release([p for p in table[keep:] if p != UNMAPPED])
            del table[keep:]
            self._table_rows[gi][r.slot, keep:] = UNMAPPED
        r.length = length
        r.reserved = min(r.reserved, keep * self.page_size)

    def block_table(self, rid: Hashable, group: int = 0) -> List[int]:
        return self._requests[rid].tables[group]

    def table_rows(self, group: int = 0) -> np.ndarray:
        """int32 [max_requests, max_blocks]: the block table of the request in each state slot
        (UNMAPPED where nothing is mapped). Read-only for callers."""
        return self._table_rows[group]

    def slot_of_position(self, rid: Hashable, group: int, position: int) -> int:
        """page * page_size + offset for a mapped position."""
        page = self._requests[rid].tables[group][position // self.page_size]
        if page == UNMAPPED:
            raise InvalidArgument(f"position {position} of request {rid!r} is not mapped in group {group}")
        return page * self.page_size + position % self.page_size

    # -- accounting -----------------------------------------------------------
    def pages_in_use(self, group: int = 0) -> int:
        return self.groups[group].pool.pages_in_use

    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.free_pages

    def check(self) -> None:
        """Invariants over pools, tables and slots (used by the tests)."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            held = [p for r in self._requests.values() for p in r.tables[gi] if p != UNMAPPED]
            assert len(held) == len(set(held)), f"group {gi}: a page is in two tables"
            assert len(held) == g.pool.pages_in_use, f"group {gi}: {g.pool.pages_in_use} pages held, tables name {len(held)}"
        slots = [r.slot for r in self._requests.values()]
        assert len(set(slots)) == len(slots), "a state slot is held twice"
        assert len(set(self._free_slots)) == len(self._free_slots)
        assert not set(slots) & set(self._free_slots), "a state slot is free and held"
        assert len(slots) + len(self._free_slots) == self.max_requests, "a state slot was lost"
