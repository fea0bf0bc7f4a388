"""A pool of equal pages and the invariant that every page is in exactly one place.

Pure Python, no tensors: this decides WHICH pages a request holds; ``cache/storage.py`` owns the
memory.  Behaviour follows ved1beta/nanospec kv/allocator.py:21-85: the free list hands out page 0
first and takes freed pages back on top, so the pages a finished request gave back are the next
ones handed out (:27,46,72); running out raises before anything is changed (:44-45).
"""

from __future__ import annotations


class PoolExhausted(Exception):
    """More pages (or state slots) were asked for than are free.  Nothing was changed."""


class PagePool:
    def __init__(self, num_pages: int, page_size: int) -> None:
        if num_pages <= 0 or page_size <= 0:
            raise ValueError(f"a pool needs pages and a page size, got {num_pages} x {page_size}")
        self.num_pages, self.page_size = num_pages, page_size
        self._free: list[int] = list(range(num_pages - 1, -1, -1))
        self._is_free = [True] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def take(self, n: int) -> list[int]:
        if n > len(self._free):
            raise PoolExhausted(f"{n} pages wanted, {len(self._free)} free of {self.num_pages}")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._is_free[p] = False
        return out

    def give(self, pages) -> None:
        pages = list(pages)
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} is not of this pool")
            if self._is_free[p]:
                raise ValueError(f"page {p} is given back twice")
        if len(set(pages)) != len(pages):
            raise ValueError(f"a page is given back twice in {pages}")
        for p in pages:
            self._is_free[p] = True
        self._free.extend(pages)

    def free_pages(self) -> list[int]:
        return list(self._free)


class SlotPool:
    """Fixed-size per-request state lives in numbered slots; same discipline as pages."""

    def __init__(self, num_slots: int) -> None:
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._is_free = [True] * num_slots

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise PoolExhausted(f"all {self.num_slots} state slots are held")
        s = self._free.pop()
        self._is_free[s] = False
        return s

    def give(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or self._is_free[slot]:
            raise ValueError(f"state slot {slot} is not held")
        self._is_free[slot] = True
        self._free.append(slot)

    def free_slots(self) -> list[int]:
        return list(self._free)
