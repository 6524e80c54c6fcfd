"""The cache manager: which pages and which slot each live request holds.

This is policy on the host; the memory itself is device tensors that the
engine owns.  Layers with the same needs form a *group* (all keys; or a window
of the last W keys).  Each group has a page pool of its own and each request
has one block table per group, shared by all layers of the group: page id p
addresses the same place in every layer's tensor, as one block id does in the
reference's pool (backend/model.cu:41, :1096-1097).

Protocol, as in the reference (engine/kv/kv.go:51-74, engine/engine.go:160-185):
``reserve(request, n)`` makes room for n more tokens, the step runs,
``commit(request, n)`` records them.  Unlike the reference's Reserve, which
keeps the pages it got before it ran out (engine/kv/kv.go:52-53), a
reservation here is all or nothing across every group.

Pages are given back when a request is released, and, in a windowed group,
as soon as every position of a page lies behind the window of every token
still to come.  Pages are not cleared when they are handed out again; readers
never look beyond a request's own length.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

from .pages import CacheError, OutOfPages, PagePool, SlotPool

FREED = -1


@dataclass(frozen=True)
class GroupSpec:
    """One group of layers with the same cache needs."""
    name: str
    page_size: int
    num_pages: int
    window: int = 0  # 0: all keys are kept


def window_pages(n_tokens: int, step_tokens: int, page_size: int, window: int) -> int:
    """Most pages a request of up to n_tokens holds in a group: all of its
    pages without a window; with one, the pages from the first key that the
    oldest token still to come may read to the end of the step being reserved:
    at most ceil((step + window - 1) / page_size) + 1."""
    whole = -(-n_tokens // page_size)
    if window <= 0:
        return whole
    return min(whole, -(-(step_tokens + window - 1) // page_size) + 1)


@dataclass
class RequestCache:
    request_id: Hashable
    slot: int
    length: int = 0                                   # tokens committed
    reserved: int = 0                                 # tokens reserved beyond length
    tables: List[List[int]] = field(default_factory=list)   # per group, logical order
    first_live: List[int] = field(default_factory=list)     # per group: first page not freed


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], num_slots: int):
        self.groups = list(groups)
        self.pools = [PagePool(g.num_pages, g.page_size) for g in self.groups]
        self.slots = SlotPool(num_slots)
        self.requests: Dict[Hashable, RequestCache] = {}

    # ------------------------------------------------------------ requests
    def open(self, request_id: Hashable) -> RequestCache:
        """A new request: takes a state slot, holds no pages yet."""
        if request_id in self.requests:
            raise CacheError(f"request {request_id!r} is already open")
        slot = self.slots.alloc()
        rc = RequestCache(request_id, slot, tables=[[] for _ in self.groups],
                          first_live=[0 for _ in self.groups])
        self.requests[request_id] = rc
        return rc

    def get(self, request_id: Hashable) -> RequestCache:
        try:
            return self.requests[request_id]
        except KeyError:
            raise CacheError(f"request {request_id!r} is not open") from None

    def __contains__(self, request_id):
        return request_id in self.requests

    # ------------------------------------------------------------ sizes
    def _first_needed_page(self, g: int, length: int) -> int:
        """First page of group g that a token at position >= length can still
        read.  A token at position p reads keys (p - window, p]."""
        w = self.groups[g].window
        if w <= 0:
            return 0
        lowest = length - w + 1
        return max(0, lowest) // self.groups[g].page_size

    def pages_needed(self, request_id: Hashable, n_tokens: int) -> List[int]:
        """New pages per group that reserving n_tokens more would take."""
        rc = self.get(request_id)
        need = []
        for g, grp in enumerate(self.groups):
            total = -(-(rc.length + rc.reserved + n_tokens) // grp.page_size)
            need.append(max(0, total - len(rc.tables[g])))
        return need

    def can_reserve(self, request_id: Hashable, n_tokens: int) -> bool:
        need = self.pages_needed(request_id, n_tokens)
        return all(n <= p.free_pages for n, p in zip(need, self.pools))

    def pages_for_tokens(self, n_tokens: int, step_tokens: Optional[int] = None) -> List[int]:
        """Pages per group that a request growing to n_tokens holds at most at
        one time, when no step brings it more than ``step_tokens`` tokens
        (default: all of them at once).  A windowed group never holds more
        than its window and one step's tokens span."""
        step = n_tokens if step_tokens is None else max(1, min(int(step_tokens), n_tokens))
        return [window_pages(n_tokens, step, grp.page_size, grp.window) for grp in self.groups]

    # ------------------------------------------------------------ protocol
    def reserve(self, request_id: Hashable, n_tokens: int) -> None:
        """Room for n_tokens more, in every group, or OutOfPages and nothing taken."""
        if n_tokens <= 0:
            raise ValueError("reserve needs a positive token count")
        rc = self.get(request_id)
        need = self.pages_needed(request_id, n_tokens)
        for g, n in enumerate(need):
            if n > self.pools[g].free_pages:
                raise OutOfPages(
                    f"request {request_id!r}: group {self.groups[g].name!r} needs {n} more "
                    f"pages for {n_tokens} tokens, {self.pools[g].free_pages} are free")
        for g, n in enumerate(need):
            rc.tables[g].extend(self.pools[g].alloc(n))
        rc.reserved += n_tokens

    def cancel(self, request_id: Hashable) -> None:
        """Undo reservations that were not committed (a step that failed)."""
        rc = self.get(request_id)
        rc.reserved = 0
        for g, grp in enumerate(self.groups):
            keep = -(-rc.length // grp.page_size)
            extra = rc.tables[g][keep:]
            del rc.tables[g][keep:]
            self.pools[g].free([p for p in extra if p != FREED])

    def commit(self, request_id: Hashable, n_tokens: int) -> None:
        """n_tokens were written.  Pages that now lie wholly behind a window
        are given back."""
        rc = self.get(request_id)
        if n_tokens <= 0 or n_tokens > rc.reserved:
            raise CacheError(
                f"request {request_id!r}: commit of {n_tokens} tokens, {rc.reserved} reserved")
        rc.length += n_tokens
        rc.reserved -= n_tokens
        for g in range(len(self.groups)):
            first = min(self._first_needed_page(g, rc.length), len(rc.tables[g]))
            if first > rc.first_live[g]:
                gone = rc.tables[g][rc.first_live[g]:first]
                self.pools[g].free(gone)
                for j in range(rc.first_live[g], first):
                    rc.tables[g][j] = FREED
                rc.first_live[g] = first

    def release(self, request_id: Hashable) -> None:
        """The request is over: every page and its slot go back."""
        rc = self.get(request_id)
        for g in range(len(self.groups)):
            self.pools[g].free([p for p in rc.tables[g] if p != FREED])
        self.slots.free(rc.slot)
        del self.requests[request_id]

    # ------------------------------------------------------------ views
    def table(self, request_id: Hashable, group: int) -> List[int]:
        return self.get(request_id).tables[group]

    def stats(self) -> dict:
        return {
            "live_requests": len(self.requests),
            "free_slots": self.slots.free_slots,
            "groups": [
                {"name": g.name, "page_size": g.page_size, "window": g.window,
                 "pages": p.num_pages, "used": p.used_pages, "free": p.free_pages,
                 "high_water": p.high_water}
                for g, p in zip(self.groups, self.pools)],
        }

    def check_invariants(self) -> None:
        """No page lost, none held twice: used for tests and debugging."""
        for g, pool in enumerate(self.pools):
            seen = set()
            for rc in self.requests.values():
                for p in rc.tables[g]:
                    if p == FREED:
                        continue
                    if p in seen:
                        raise CacheError(f"group {g}: page {p} is in two tables")
                    if not pool.is_held(p):
                        raise CacheError(f"group {g}: page {p} is in a table but free")
                    seen.add(p)
            if len(seen) != pool.used_pages:
                raise CacheError(
                    f"group {g}: {pool.used_pages} pages are out, tables hold {len(seen)}")
            if len(set(pool._free)) != len(pool._free):
                raise CacheError(f"group {g}: a page is twice in the free list")
