"""Pages and slots: the two pools the cache manager hands out from.

``PagePool`` follows the reference's allocator (engine/kv/kv.go:9-40): a
last-in-first-out free list of int32 page ids, filled so that low ids are
handed out first; pages come back in the order given.  It adds what the
reference leaves to trust: an allocation of several pages is all or nothing,
and a page that is freed twice or was never handed out is an error.
"""

from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """The pool cannot cover a reservation."""


class CacheError(RuntimeError):
    """A misuse of the cache manager: an unknown request, a double free."""


class PagePool:
    def __init__(self, num_pages: int, page_size: int):
        if num_pages < 0 or page_size <= 0:
            raise ValueError(f"bad pool: {num_pages} pages of {page_size} tokens")
        self.num_pages = num_pages
        self.page_size = page_size
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages
        self.high_water = 0
        self.total_allocs = 0

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def used_pages(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self, n: int) -> List[int]:
        """n pages or none: raises OutOfPages and takes nothing if fewer are free."""
        if n < 0:
            raise ValueError("negative page count")
        if n > len(self._free):
            raise OutOfPages(
                f"need {n} pages, {len(self._free)} of {self.num_pages} are free")
        ids = [self._free.pop() for _ in range(n)]
        for i in ids:
            self._held[i] = True
        self.total_allocs += n
        self.high_water = max(self.high_water, self.used_pages)
        return ids

    def free(self, ids) -> None:
        ids = list(ids)
        for i in ids:
            if not 0 <= i < self.num_pages:
                raise CacheError(f"page {i} does not belong to this pool")
            if not self._held[i]:
                raise CacheError(f"page {i} freed twice")
            self._held[i] = False
        self._free.extend(ids)

    def is_held(self, page: int) -> bool:
        return self._held[page]


class SlotPool:
    """Slots for per-request state of fixed size: one per live request."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = [False] * num_slots

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages(f"all {self.num_slots} state slots are taken")
        s = self._free.pop()
        self._held[s] = True
        return s

    def free(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or not self._held[slot]:
            raise CacheError(f"slot {slot} freed twice or never taken")
        self._held[slot] = False
        self._free.append(slot)
