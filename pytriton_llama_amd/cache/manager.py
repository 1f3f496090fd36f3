"""The cache manager: who holds which page, and which state slot.

The reference hands out single token slots from a reference-count vector on the
GPU, reserves batch x (prompt + max_gen) of them before the first forward and
gives them back when the whole batch is done
(lite_llama/executor/mem_manager.py:134-263, lite_llama/generate_stream.py:136,188).
Here the unit is a page of ``page_size`` tokens, pages are taken when a request's
tokens need them and go back on the free list when the request ends or, for a
group with a window, when every later query has moved past them. All of it is
host-side bookkeeping: no device call, no synchronisation.

Cache layers with the same needs form a group; a group has a page pool and, for
every live request, a block table of its own. Beside the pages every live
request owns one state slot 0..max_num_seqs-1: the row of the device block
tables and of every fixed-size state tensor that belongs to it. One more slot,
``padding_slot`` = max_num_seqs, belongs to nobody: rows that pad a step to the size of a
recorded graph name it, so that a mixer with state reads and writes there and harms no request.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from ..parts.base import PagedSpec, StateSpec

RELEASED = -1   # block-table entry of a page that was given back (left of the window)


class OutOfPages(RuntimeError):
    """A request needs more pages than are free."""


class OutOfSlots(RuntimeError):
    """More live requests than state slots."""


class PagePool:
    """Free list (LIFO) of page ids 0..num_pages-1 with a held/free flag per page."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = int(num_pages)
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))
        self._held = [False] * self.num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def give_back(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not (0 <= p < self.num_pages) or not self._held[p]:
                raise RuntimeError(f"page {p} given back but not held")
            self._held[p] = False
            self._free.append(p)

    def is_held(self, p: int) -> bool:
        return self._held[p]


@dataclass
class PagedGroup:
    spec: PagedSpec
    layers: List[int]                 # cache-layer ids stored in this group, in order
    page_size: int
    pool: PagePool
    tables: Dict[Hashable, List[int]] = field(default_factory=dict)

    def first_needed_page(self, num_tokens: int) -> int:
        """Index of the first page a query at position >= num_tokens can read."""
        if self.spec.window is None:
            return 0
        return max(0, num_tokens - self.spec.window + 1) // self.page_size


@dataclass
class StateGroup:
    spec: StateSpec
    layers: List[int]


class CacheManager:
    def __init__(self, cache_layers: Sequence[object], page_size: int, num_pages,
                 max_num_seqs: int):
        """cache_layers: one PagedSpec / StateSpec / None per cache layer of the
        model. num_pages: an int (every paged group gets that many) or one int
        per paged group."""
        if page_size <= 0 or max_num_seqs <= 0:
            raise ValueError("page_size and max_num_seqs must be positive")
        self.page_size = int(page_size)
        self.max_num_seqs = int(max_num_seqs)
        self.paged: List[PagedGroup] = []
        self.states: List[StateGroup] = []
        self.layer_home: List[Optional[Tuple[str, int, int]]] = []   # (kind, group, index in group)
        by_spec: Dict[object, Tuple[str, int]] = {}
        for lid, spec in enumerate(cache_layers):
            if spec is None:
                self.layer_home.append(None)
                continue
            if spec not in by_spec:
                if isinstance(spec, PagedSpec):
                    by_spec[spec] = ("paged", len(self.paged))
                    self.paged.append(PagedGroup(spec, [], self.page_size, None))
                elif isinstance(spec, StateSpec):
                    by_spec[spec] = ("state", len(self.states))
                    self.states.append(StateGroup(spec, []))
                else:
                    raise TypeError(f"cache layer {lid}: unknown cache spec {spec!r}")
            kind, g = by_spec[spec]
            group = self.paged[g] if kind == "paged" else self.states[g]
            self.layer_home.append((kind, g, len(group.layers)))
            group.layers.append(lid)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(self.paged)
        if len(num_pages) != len(self.paged):
            raise ValueError(f"{len(self.paged)} paged groups but {len(num_pages)} pool sizes")
        for g, n in zip(self.paged, num_pages):
            g.pool = PagePool(n)
        self._free_slots: List[int] = list(range(self.max_num_seqs - 1, -1, -1))
        self.padding_slot = self.max_num_seqs        # the state row of rows that pad a step
        self.slot_of: Dict[Hashable, int] = {}
        self.num_tokens: Dict[Hashable, int] = {}

    # ---- requests ------------------------------------------------------------
    def is_live(self, req) -> bool:
        return req in self.slot_of

    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self, req) -> int:
        """Give ``req`` a state slot and empty block tables."""
        if req in self.slot_of:
            raise RuntimeError(f"request {req!r} is already live")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.max_num_seqs} state slots are taken")
        slot = self._free_slots.pop()
        self.slot_of[req] = slot
        self.num_tokens[req] = 0
        for g in self.paged:
            g.tables[req] = []
        return slot

    def pages_needed(self, req, n_new: int) -> List[int]:
        """Pages each paged group must take so that ``req`` can hold n_new more
        tokens (a request not yet admitted counts from zero)."""
        have = self.num_tokens.get(req, 0)
        total = -(-(have + n_new) // self.page_size)
        return [max(0, total - len(g.tables.get(req, ()))) for g in self.paged]

    def can_append(self, req, n_new: int, reserve: Optional[Sequence[int]] = None) -> bool:
        """``reserve``: pages per group already promised to others in this pass."""
        need = self.pages_needed(req, n_new)
        for i, (g, n) in enumerate(zip(self.paged, need)):
            if n + (reserve[i] if reserve else 0) > g.pool.num_free:
                return False
        return True

    def append(self, req, n_new: int) -> int:
        """Take the pages for n_new more tokens of ``req``; returns the position
        of the first of them. Takes nothing if any group cannot serve it."""
        if req not in self.slot_of:
            raise RuntimeError(f"request {req!r} is not live")
        if n_new <= 0:
            raise ValueError("append needs at least one token")
        need = self.pages_needed(req, n_new)
        for g, n in zip(self.paged, need):
            if n > g.pool.num_free:
                raise OutOfPages(f"request {req!r} needs {n} more pages of {g.spec}, "
                                 f"{g.pool.num_free} free")
        for g, n in zip(self.paged, need):
            g.tables[req].extend(g.pool.take(n))
        start = self.num_tokens[req]
        self.num_tokens[req] = start + n_new
        return start

    def slot_array(self, req, group: int, start: int, n: int) -> np.ndarray:
        """Flat cache slots page*page_size+offset of positions start..start+n-1 (int32)."""
        table = self.paged[group].tables[req]
        P = self.page_size
        first = start // P
        pages = np.asarray(table[first:(start + n - 1) // P + 1], dtype=np.int64)
        if n <= 0 or pages.size != (start + n - 1) // P + 1 - first:
            raise RuntimeError(f"request {req!r}: positions {start}..{start + n - 1} lie outside its pages")
        if (pages < 0).any():
            pos = (first + int(np.argmax(pages < 0))) * P
            raise RuntimeError(f"request {req!r}: position {max(pos, start)} lies in a released page")
        pos = np.arange(start, start + n, dtype=np.int64)
        return (pages[pos // P - first] * P + pos % P).astype(np.int32)

    def slots(self, req, group: int, start: int, n: int) -> List[int]:
        """The same as a list."""
        return self.slot_array(req, group, start, n).tolist()

    def release_behind_window(self, req) -> int:
        """Give back the pages of ``req`` that no later query can read (groups
        with a window only). Their table entries become RELEASED. Returns the
        number of pages given back."""
        n = 0
        have = self.num_tokens[req]
        for g in self.paged:
            if g.spec.window is None:
                continue
            table = g.tables[req]
            first = min(g.first_needed_page(have), len(table))
            dead = [table[i] for i in range(first) if table[i] >= 0]
            if dead:
                g.pool.give_back(dead)
                for i in range(first):
                    table[i] = RELEASED
                n += len(dead)
        return n

    def free(self, req) -> None:
        """The request is over: its pages and its slot go back."""
        if req not in self.slot_of:
            raise RuntimeError(f"request {req!r} is not live (freed twice?)")
        for g in self.paged:
            g.pool.give_back([p for p in g.tables.pop(req) if p >= 0])
        self._free_slots.append(self.slot_of.pop(req))
        del self.num_tokens[req]

    def block_table(self, req, group: int) -> List[int]:
        return self.paged[group].tables[req]

    # ---- checks (used by tests and debug runs) ---------------------------------
    def check(self) -> None:
        """No page lost, held twice or free while in a table; slots likewise."""
        for gi, g in enumerate(self.paged):
            seen = {}
            for req, table in g.tables.items():
                for p in table:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError(f"group {gi}: page {p} held by {seen[p]!r} and {req!r}")
                    if not g.pool.is_held(p):
                        raise AssertionError(f"group {gi}: page {p} of {req!r} is on the free list")
                    seen[p] = req
            if len(seen) + g.pool.num_free != g.pool.num_pages:
                raise AssertionError(f"group {gi}: {len(seen)} held + {g.pool.num_free} free "
                                     f"!= {g.pool.num_pages} pages")
            if len(set(g.pool._free)) != len(g.pool._free):
                raise AssertionError(f"group {gi}: a page is on the free list twice")
        slots = list(self.slot_of.values())
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots) \
                or len(slots) + len(self._free_slots) != self.max_num_seqs:
            raise AssertionError("state slots are inconsistent")
