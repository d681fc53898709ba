"""One group's pages: who holds them, which are free, which are kept for reuse by content.

A page is in exactly one state (reference: src/dli/kv/block_manager.py:9-15):
FREE (on the free list), USED (held by ``ref`` block-table entries) or CACHED-IDLE (held by
nobody, still registered under its content identity: a later request with the same prefix can
revive it, and it is reclaimed, leaves first, when memory is needed).
"""

from __future__ import annotations

from collections import Counter, deque
from dataclasses import dataclass
from typing import Optional

from .reclaim import ReclaimOrder, make_order
from .page_identity import PageHash


@dataclass
class _CachedPage:
    identity: PageHash
    parent: Optional[int]
    depth: int
    children: int = 0


class PagePool:
    def __init__(self, num_pages: int, eviction_policy: str | ReclaimOrder = "lru") -> None:
        if num_pages <= 0:
            raise ValueError("num_pages must be positive")
        self.num_pages = num_pages
        self.order: ReclaimOrder = (
            make_order(eviction_policy) if isinstance(eviction_policy, str) else eviction_policy
        )
        self.ref = [0] * num_pages
        self.free: deque[int] = deque(range(num_pages))
        self.cached: dict[int, _CachedPage] = {}
        self.by_identity: dict[PageHash, int] = {}
        self.num_idle = 0
        self.evictions = 0

    @property
    def num_available(self) -> int:
        """Pages obtainable now: free ones and idle cached ones."""
        return len(self.free) + self.num_idle

    def take(self) -> int:
        """A page for a new holder. Callers check :attr:`num_available` first."""
        page = self.free.popleft() if self.free else self._evict(self.order.take())
        self.ref[page] = 1
        return page

    def incref(self, page: int) -> None:
        if self.ref[page] == 0:
            entry = self.cached.get(page)
            if entry is None:
                raise AssertionError(f"page {page} is free and cannot gain a holder")
            self.num_idle -= 1
            if entry.children == 0:
                self.order.withdraw(page)
        self.ref[page] += 1

    def decref(self, page: int) -> None:
        if self.ref[page] <= 0:
            raise AssertionError(f"page {page} is given back twice")
        self.ref[page] -= 1
        if self.ref[page] > 0:
            return
        entry = self.cached.get(page)
        if entry is None:
            self.free.append(page)
            return
        self.num_idle += 1
        if entry.children == 0:
            self.order.offer(page)

    def _evict(self, page: int) -> int:
        entry = self.cached.pop(page)
        del self.by_identity[entry.identity]
        self.num_idle -= 1
        self.order.dropped(page)
        self.evictions += 1
        if entry.parent is not None:
            parent = self.cached[entry.parent]
            parent.children -= 1
            if parent.children == 0 and self.ref[entry.parent] == 0:
                self.order.offer(entry.parent)
        return page

    def evict_all_idle(self) -> int:
        n = 0
        while len(self.order):
            self.free.append(self._evict(self.order.take()))
            n += 1
        return n

    def register(self, page: int, identity: PageHash, parent_identity: Optional[PageHash],
                 parent_page: Optional[int], depth: int) -> str:
        """Enter a full, computed page into the content index.

        Returns ``"cached"``, ``"already"`` (the page is in the index), ``"duplicate"`` (the same
        content is cached in another page: this one stays private) or ``"orphan"`` (its parent is
        not this request's own cached page, so linking it would break the closed-prefix rule;
        reference: src/dli/kv/block_manager.py:538-562).
        """
        if page in self.cached:
            return "already"
        if identity in self.by_identity:
            return "duplicate"
        parent: Optional[int] = None
        if parent_identity is not None:
            parent = self.by_identity.get(parent_identity)
            if parent is None or parent != parent_page:
                return "orphan"
            pentry = self.cached[parent]
            if pentry.children == 0 and self.ref[parent] == 0:
                self.order.withdraw(parent)
            pentry.children += 1
        self.cached[page] = _CachedPage(identity, parent, depth)
        self.by_identity[identity] = page
        self.order.cached(page, depth)
        return "cached"

    def check(self, expected_ref: Counter) -> None:
        """Raise AssertionError at the first inconsistency (reference:
        src/dli/kv/block_manager.py:384-433)."""
        for p in range(self.num_pages):
            assert self.ref[p] == expected_ref[p], f"page {p}: ref {self.ref[p]} != {expected_ref[p]} holders"
        free = set(self.free)
        assert len(free) == len(self.free), "a page is on the free list twice"
        cached = set(self.cached)
        used = {p for p in range(self.num_pages) if self.ref[p] > 0}
        assert not free & cached, "a page is both free and cached"
        assert not free & used, "a page is both free and held"
        assert free | cached | used == set(range(self.num_pages)), "a page is in no state (lost)"
        idle = cached - used
        assert len(idle) == self.num_idle, "idle counter drifted"
        assert len(self.by_identity) == len(self.cached), "content index size mismatch"
        children: Counter = Counter()
        for p, e in self.cached.items():
            assert self.by_identity.get(e.identity) == p, f"page {p} is not indexed by its identity"
            if e.parent is not None:
                assert e.parent in self.cached, f"page {p}: parent not cached (prefix not closed)"
                children[e.parent] += 1
        for p, e in self.cached.items():
            assert e.children == children[p], f"page {p}: children {e.children} != {children[p]}"
        for p in cached & used:
            parent = self.cached[p].parent
            assert parent is None or self.ref[parent] > 0, f"held page {p} has an idle parent"
        candidates = {p for p in idle if self.cached[p].children == 0}
        assert len(self.order) == len(candidates), (
            f"the reclaim order holds {len(self.order)} candidates, expected {len(candidates)}")
