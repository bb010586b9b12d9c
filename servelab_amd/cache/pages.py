"""Free list of physical pages and free list of state slots.

Reference: ``BlockManager.free_ids`` is ``deque(range(num_blocks))``, pages are
taken with ``popleft`` and given back with ``extend`` (FIFO reuse,
servelab/kv_cache/manager.py:42,187-190,226).  A page held twice or freed
twice is an error here instead of silent corruption.
"""
from collections import deque
from typing import Hashable, List, Optional


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("num_pages must be >= 1")
        self.num_pages = int(num_pages)
        self._free = deque(range(self.num_pages))
        self._held = [False] * self.num_pages
        self.alloc_fails = 0
        self.high_water = 0

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def take(self, n: int) -> Optional[List[int]]:
        """``n`` pages, or None (and nothing taken) when fewer are free."""
        if n > len(self._free):
            self.alloc_fails += 1
            return None
        pages = [self._free.popleft() for _ in range(n)]
        for p in pages:
            if self._held[p]:
                raise AssertionError(f"page {p} handed out while held")
            self._held[p] = True
        self.high_water = max(self.high_water, self.num_used)
        return pages

    def give(self, pages) -> None:
        for p in pages:
            if not (0 <= p < self.num_pages) or not self._held[p]:
                raise AssertionError(f"page {p} freed while not held")
            self._held[p] = False
            self._free.append(p)

    def is_held(self, page: int) -> bool:
        return self._held[page]


class SlotAllocator:
    """Slots for per-request state of fixed size: one slot per live request."""

    def __init__(self, num_slots: int):
        self.num_slots = int(num_slots)
        self._free = deque(range(self.num_slots))
        self._owner: dict = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, request: Hashable) -> Optional[int]:
        if request in self._owner:
            raise AssertionError(f"request {request!r} already holds a state slot")
        if not self._free:
            return None
        slot = self._free.popleft()
        self._owner[request] = slot
        return slot

    def give(self, request: Hashable) -> None:
        self._free.append(self._owner.pop(request))

    def slot_of(self, request: Hashable) -> int:
        return self._owner[request]

    def owners(self):
        return dict(self._owner)
