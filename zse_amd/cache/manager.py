"""The cache manager: pages per group of layers, a block table per request
and group, and the request's state slot.

Groups.  Entries of the execution order whose mixers keep keys and values fall
into groups by what they need: every key ever written, or only a window of
them.  Each group has a pool of its own and each request one block table per
group; a page id names the same place in the slab of every layer of its
group.  The reference has one pool whose block holds all layers, and trims a
window for all layers at once while shortening the sequence length
(cache/cache_manager.py:265-267, 405-428; cache/page_table.py:191-194); here a
release never changes a request's length and concerns the windowed group only.

Tables.  Entry j of a request's table covers positions [j*page, (j+1)*page);
entries whose page was given back read -1 (holes, as cache/page_table.py:115-128).

Reservation is per step and all-or-nothing (the reference reserves the whole
prompt up front, cache/cache_manager.py:185-234): ``reserve(req, upto)``
makes sure every group has pages for positions below ``upto``.
``commit(req, n)`` records that n tokens are computed and gives back, in
windowed groups, each page j with (j+1)*page - 1 <= n - window: its newest key
is out of sight of every query at position >= n.  ``release(req)`` gives
everything back; a second call does nothing (double free is a no-op,
cache/cache_manager.py:269-283).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np

from .pages import OutOfPages, PagePool
from .slots import OutOfSlots, StateSlots


@dataclass
class GroupInfo:
    window: Optional[int]          # None: keeps every key
    calls: List[int]               # entries of the execution order in this group
    num_pages: int = 0


@dataclass
class _Req:
    slot: int
    computed: int = 0                                   # tokens whose keys are in the cache
    tables: List[List[int]] = field(default_factory=list)   # per group, page ids or -1
    first_live: List[int] = field(default_factory=list)      # per group, first table entry still held


def group_needs(needs: Sequence[object]) -> List[GroupInfo]:
    """Group the paged needs of an execution order by their window."""
    from ..parts.base import PagedKV
    groups: Dict[Optional[int], GroupInfo] = {}
    for i, n in enumerate(needs):
        if isinstance(n, PagedKV):
            groups.setdefault(n.window, GroupInfo(n.window, [])).calls.append(i)
    # windowed groups first, by window; the all-keys group last
    return sorted(groups.values(), key=lambda g: (g.window is None, g.window or 0))


class CacheManager:
    def __init__(self, groups: Sequence[GroupInfo], page_size: int, max_seqs: int,
                 max_model_len: int, slot_bytes: int = 0, first_page: int = 0):
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.page_size = int(page_size)
        self.groups = list(groups)
        # first_page = 1: the owner of the slabs keeps page 0 of every slab to itself (cleared,
        # never handed out), which is what a kernel reads for a table entry without a page
        self.pools = [PagePool(g.num_pages, first_page) for g in self.groups]
        self.slots = StateSlots(max_seqs, slot_bytes)
        self.max_model_len = int(max_model_len)
        self.max_blocks = -(-self.max_model_len // self.page_size)
        self._reqs: Dict[object, _Req] = {}
        # called with (request, slot) whenever a request becomes live, whoever admits it (a
        # scheduler, a step that meets a new request, a request computed again after giving
        # everything up): the owner of the slots' memory clears the slot here
        self.on_admit: Optional[Callable[[object, int], None]] = None

    # ---- requests
    def add(self, req) -> int:
        """Admit a request: it gets a state slot (raises ``OutOfSlots``), and the slot's
        memory is cleared through ``on_admit``.  This is the only way a request becomes live."""
        if req in self._reqs:
            raise ValueError(f"request {req!r} is already live")
        slot = self.slots.acquire(req)
        self._reqs[req] = _Req(slot, 0, [[] for _ in self.groups], [0 for _ in self.groups])
        if self.on_admit is not None:
            self.on_admit(req, slot)
        return slot

    def has(self, req) -> bool:
        return req in self._reqs

    def live(self) -> List[object]:
        return list(self._reqs)

    def slot(self, req) -> int:
        return self._reqs[req].slot

    def computed(self, req) -> int:
        return self._reqs[req].computed

    # ---- pages
    def pages_short(self, req, upto: int) -> List[int]:
        """Per group: how many more pages ``reserve(req, upto)`` would need than are free."""
        r = self._reqs[req]
        want = -(-upto // self.page_size)
        return [max(0, want - len(r.tables[g]) - self.pools[g].free_pages)
                for g in range(len(self.groups))]

    def reserve(self, req, upto: int) -> bool:
        """Pages for every position below ``upto`` in every group, or none at all."""
        if upto > self.max_model_len:
            raise ValueError(f"request {req!r} would reach {upto} tokens; the limit is "
                             f"{self.max_model_len}")
        r = self._reqs[req]
        want = -(-upto // self.page_size)
        tables = r.tables
        if all(len(t) >= want for t in tables):      # the usual case: the last page has room
            return True
        need = [max(0, want - len(t)) for t in tables]
        if any(need[g] > self.pools[g].free_pages for g in range(len(self.groups))):
            return False
        for g, n in enumerate(need):
            for _ in range(n):
                tables[g].append(self.pools[g].alloc(req))
        return True

    def commit(self, req, computed: int) -> List[List[int]]:
        """Record the request's computed length; return the pages given back per group."""
        r = self._reqs[req]
        if computed < r.computed:
            raise ValueError("a request's computed length never shrinks")
        r.computed = computed
        freed = []
        ps = self.page_size
        for g, info in enumerate(self.groups):
            out = []
            if info.window is not None:
                t = r.tables[g]
                j = r.first_live[g]
                while j < len(t) and (j + 1) * ps - 1 <= computed - info.window:
                    if t[j] >= 0:
                        self.pools[g].free(t[j], req)
                        out.append(t[j])
                        t[j] = -1
                    j += 1
                r.first_live[g] = j
            freed.append(out)
        return freed

    def release(self, req) -> None:
        r = self._reqs.pop(req, None)
        if r is None:
            return
        for g, t in enumerate(r.tables):
            for p in t:
                if p >= 0:
                    self.pools[g].free(p, req)
        self.slots.release(req)

    # ---- what a step needs
    def untouched_page(self, req, group: int, upto: int) -> Optional[int]:
        """The page that a step bringing the request to ``upto`` tokens begins to fill without
        filling it: its id, if the request has not written to it before (it then still holds
        what its last owner left), else None.  Pages are filled in the order of positions, so
        a page is untouched exactly when all its positions lie at or behind the computed
        length; a step fills every such page but, at most, the last."""
        if upto % self.page_size == 0:
            return None
        r = self._reqs[req]
        j = (upto - 1) // self.page_size
        if j * self.page_size < r.computed:
            return None
        page = r.tables[group][j]
        return page if page >= 0 else None

    def table(self, req, group: int) -> List[int]:
        return self._reqs[req].tables[group]

    def fill_table_row(self, req, group: int, row: np.ndarray) -> None:
        t = self._reqs[req].tables[group]
        row[:len(t)] = t
        row[len(t):] = -1

    def slot_of(self, req, group: int, pos: int) -> int:
        """page * page_size + offset for one position (a decoded token's: no arrays)."""
        page = self._reqs[req].tables[group][pos // self.page_size]
        if page < 0:
            raise RuntimeError(f"request {req!r}: a position to be written lies on a released page")
        return page * self.page_size + pos % self.page_size

    def slot_mapping(self, req, group: int, start: int, n: int) -> np.ndarray:
        """page * page_size + offset for positions start .. start+n-1."""
        t = self._reqs[req].tables[group]
        pos = np.arange(start, start + n)
        pages = np.asarray(t, dtype=np.int64)[pos // self.page_size]
        if (pages < 0).any():
            raise RuntimeError(f"request {req!r}: a position to be written lies on a released page")
        return (pages * self.page_size + pos % self.page_size).astype(np.int32)

    # ---- invariants (tests)
    def check(self) -> None:
        for pool in self.pools:
            pool.check()
        self.slots.check()
        for g, pool in enumerate(self.pools):
            held = {}
            for req, r in self._reqs.items():
                for p in r.tables[g]:
                    if p >= 0:
                        if p in held:
                            raise AssertionError(f"group {g}: page {p} held by {held[p]!r} and {req!r}")
                        held[p] = req
                        if pool.owner(p) != req:
                            raise AssertionError(f"group {g}: page {p} in {req!r}'s table is owned by "
                                                 f"{pool.owner(p)!r}")
            if len(held) != pool.used_pages:
                raise AssertionError(f"group {g}: {pool.used_pages} pages are out, {len(held)} are in tables")

    def stats(self) -> dict:
        return {"page_size": self.page_size,
                "groups": [{"window": g.window, "calls": len(g.calls), "pages": p.num_pages,
                            "free": p.free_pages} for g, p in zip(self.groups, self.pools)],
                "live": len(self._reqs), "free_slots": self.slots.free_slots}
