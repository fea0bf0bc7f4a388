"""The cache manager: block tables per request and per group of layers, and state slots.

Layers whose mixers keep the same kind of cache form a GROUP with pages of its own: all keys and
values of a request (``window == 0``), or only the last ``window`` positions, in which case pages
that have fallen out of the window are given back while the request is still running.  Every live
request also holds one slot for state of fixed size (used by mixers that carry a state instead of
keys; a request holds its slot even if no layer has such state).

Reference for the page bookkeeping: ved1beta/nanospec kv/allocator.py (block table = list of pages
+ a length, pages added only when a page boundary is crossed :50-58, all pages returned when the
request ends :70-74, ``check()`` :79-85).  Groups, windows and state slots are not in the reference.

Two lengths per request: ``reserved`` positions have a page in every group; ``length`` positions
have been written by a step.  ``reserve(n)`` makes ``reserved >= length + n`` (and is the only call
that can run out of pages; it changes nothing when it does), ``commit`` grows ``length`` and lets
windows let go.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .pages import PagePool, PoolExhausted, SlotPool

RELEASED = -1  # block-table entry of a page that a window has let go


@dataclass(frozen=True)
class GroupSpec:
    """What one group of layers keeps per token.  ``window`` = 0 keeps everything."""

    name: str
    window: int = 0


@dataclass
class RequestCache:
    req_id: object
    slot: int
    tables: list[list[int]]  # per group: page of positions [i*page, (i+1)*page), or RELEASED
    reserved: int = 0
    length: int = 0
    first_kept: list[int] = field(default_factory=list)  # per group: first table index not released
    held: list[int] = field(default_factory=list)  # per group: pages held now


class CacheManager:
    def __init__(self, groups: list[GroupSpec], num_pages: int | list[int], page_size: int, num_slots: int) -> None:
        self.groups = list(groups)
        counts = num_pages if isinstance(num_pages, (list, tuple)) else [num_pages] * len(self.groups)
        if len(counts) != len(self.groups):
            raise ValueError("one page count per group is wanted")
        self.page_size = page_size
        self.pools = [PagePool(n, page_size) for n in counts]
        self.slots = SlotPool(num_slots)
        self._live: dict[object, RequestCache] = {}

    # ------------------------------------------------------------------ queries

    def __contains__(self, req_id) -> bool:
        return req_id in self._live

    def get(self, req_id) -> RequestCache:
        return self._live[req_id]

    @property
    def live(self) -> list:
        return list(self._live)

    def num_free(self, group: int = 0) -> int:
        return self.pools[group].num_free

    def pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def _first_needed_index(self, group: int, next_pos: int) -> int:
        """Index of the first table entry that a query at ``next_pos`` (and any later one) can still
        see in this group."""
        w = self.groups[group].window
        if w <= 0:
            return 0
        return max(0, next_pos - w + 1) // self.page_size

    def pages_missing(self, req_id, n_tokens: int) -> list[int]:
        """Pages each group lacks for ``length + n_tokens`` positions (what ``reserve`` would take)."""
        rc = self._live[req_id]
        want = self.pages_for(rc.length + n_tokens)
        return [max(0, want - len(t)) for t in rc.tables]

    def worst_case_pages(self, n_tokens: int) -> list[int]:
        """Most pages per group that a request of ``n_tokens`` holds at any time if it is written in
        portions of at most one page beyond a window."""
        out = []
        for g in self.groups:
            if g.window <= 0:
                out.append(self.pages_for(n_tokens))
            else:
                out.append(min(self.pages_for(n_tokens), self.pages_for(g.window) + 2))
        return out

    # ------------------------------------------------------------------ life of a request

    def admit(self, req_id) -> RequestCache:
        if req_id in self._live:
            raise ValueError(f"request {req_id!r} is already live")
        rc = RequestCache(req_id, self.slots.take(), [[] for _ in self.groups], first_kept=[0] * len(self.groups),
                          held=[0] * len(self.groups))
        self._live[req_id] = rc
        return rc

    def reserve(self, req_id, n_tokens: int) -> RequestCache:
        """Make sure positions [0, length + n_tokens) have pages in every group (asking twice for the same
        tokens takes nothing more).  Raises PoolExhausted, with nothing changed, if any group lacks them."""
        rc = self._live[req_id]
        missing = self.pages_missing(req_id, n_tokens)
        for g, need in enumerate(missing):
            if need > self.pools[g].num_free:
                raise PoolExhausted(
                    f"request {req_id!r} needs {need} more pages in group {self.groups[g].name!r}, "
                    f"{self.pools[g].num_free} free"
                )
        for g, need in enumerate(missing):
            rc.tables[g].extend(self.pools[g].take(need))
            rc.held[g] += need
        rc.reserved = max(rc.reserved, rc.length + n_tokens)
        return rc

    def commit(self, req_id, n_tokens: int) -> None:
        """``n_tokens`` more positions have been written.  Windows let go of the pages that no later
        query can see."""
        rc = self._live[req_id]
        if rc.length + n_tokens > rc.reserved:
            raise ValueError(f"request {req_id!r}: {rc.length}+{n_tokens} positions written but {rc.reserved} reserved")
        rc.length += n_tokens
        for g in range(len(self.groups)):
            keep_from = min(self._first_needed_index(g, rc.length), len(rc.tables[g]))
            gone = [p for p in rc.tables[g][rc.first_kept[g]:keep_from] if p != RELEASED]
            if gone:
                self.pools[g].give(gone)
                rc.held[g] -= len(gone)
            for i in range(rc.first_kept[g], keep_from):
                rc.tables[g][i] = RELEASED
            rc.first_kept[g] = max(rc.first_kept[g], keep_from)

    def release(self, req_id) -> None:
        """The request ends (or is preempted): every page and the state slot go back."""
        rc = self._live.pop(req_id)
        for g, table in enumerate(rc.tables):
            self.pools[g].give([p for p in table if p != RELEASED])
            table.clear()
            rc.held[g] = 0
        self.slots.give(rc.slot)
        rc.reserved = rc.length = 0

    # ------------------------------------------------------------------ invariant

    def check(self) -> None:
        """Every page of every group is free or in exactly one live table; every slot likewise;
        tables are as long as the reservation needs."""
        for g, pool in enumerate(self.pools):
            seen = pool.free_pages()
            for rc in self._live.values():
                seen.extend(p for p in rc.tables[g] if p != RELEASED)
                assert len(rc.tables[g]) == self.pages_for(rc.reserved), (rc.req_id, g, rc.tables[g], rc.reserved)
                assert all(p == RELEASED for p in rc.tables[g][: rc.first_kept[g]])
                assert all(p != RELEASED for p in rc.tables[g][rc.first_kept[g]:])
                assert rc.held[g] == sum(1 for p in rc.tables[g] if p != RELEASED)
            assert sorted(seen) == list(range(pool.num_pages)), f"group {g}: a page is lost or held twice"
        held = self.slots.free_slots() + [rc.slot for rc in self._live.values()]
        assert sorted(held) == list(range(self.slots.num_slots)), "a state slot is lost or held twice"
