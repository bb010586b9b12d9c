"""Cache manager: pages with a block table per request, in groups, and state
slots beside them.  Pure Python integers; no tensors.

Reference: ``BlockManager`` without prefix cache
(servelab/kv_cache/manager.py:153-227,306-316): one table per request serves
all layers.  Here the cache streams of a model are grouped by what they need:
streams that keep every key share one group, streams that keep a window of W
keys share another, and each group has pages and block tables of its own.  A
window group gives a page back as soon as no later query can see any of its
tokens.  Streams that need a fixed-size state per request get a slot, taken
when the request opens and given back when it closes; the slot array exists
even when no stream asks for state.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, Hashable, List, Optional

from ..parts.base import PagedKVSpec, StateSpec
from .pages import PageAllocator, SlotAllocator

RELEASED = -1      # block-table entry of a page the window has passed


@dataclass
class PageGroup:
    """Cache streams with the same page need."""
    spec: PagedKVSpec
    streams: List[int]
    allocator: PageAllocator
    tables: Dict[Hashable, List[int]] = field(default_factory=dict)

    @property
    def window(self) -> Optional[int]:
        return self.spec.window


@dataclass
class StateGroup:
    spec: StateSpec
    streams: List[int]


class CacheManager:
    def __init__(self, stream_specs: Dict[int, Any], num_pages: int, page_size: int,
                 num_state_slots: int = 64):
        self.page_size = int(page_size)
        self.num_pages = int(num_pages)
        self.page_groups: List[PageGroup] = []
        self.state_groups: List[StateGroup] = []
        self.stream_group: Dict[int, tuple] = {}      # stream -> ("pages"|"state", index, index in group)
        for stream in sorted(stream_specs):
            spec = stream_specs[stream]
            if spec is None:
                continue
            if isinstance(spec, PagedKVSpec):
                groups, kind = self.page_groups, "pages"
            elif isinstance(spec, StateSpec):
                groups, kind = self.state_groups, "state"
            else:
                raise TypeError(f"stream {stream}: unknown cache spec {spec!r}")
            for gi, g in enumerate(groups):
                if g.spec == spec:
                    break
            else:
                gi = len(groups)
                groups.append(PageGroup(spec, [], PageAllocator(num_pages)) if kind == "pages"
                              else StateGroup(spec, []))
            self.stream_group[stream] = (kind, gi, len(groups[gi].streams))
            groups[gi].streams.append(stream)
        self.state_slots = SlotAllocator(num_state_slots)
        self.lengths: Dict[Hashable, int] = {}        # tokens whose cache is written

    # ------------------------------------------------------------ requests
    def is_open(self, request) -> bool:
        return request in self.lengths

    def open(self, request) -> bool:
        """Admit a request: empty tables in every group and one state slot.
        False (nothing taken) when no slot is free."""
        if request in self.lengths:
            raise AssertionError(f"request {request!r} is already open")
        if self.state_slots.take(request) is None:
            return False
        for g in self.page_groups:
            g.tables[request] = []
        self.lengths[request] = 0
        return True

    def close(self, request) -> None:
        """Give back everything the request holds (finished, aborted or
        preempted; servelab/kv_cache/manager.py:216-227)."""
        if request not in self.lengths:
            return
        for g in self.page_groups:
            g.allocator.give([p for p in g.tables.pop(request) if p != RELEASED])
        self.state_slots.give(request)
        del self.lengths[request]

    def length(self, request) -> int:
        return self.lengths[request]

    # ------------------------------------------------------------ growing
    def pages_for(self, num_tokens: int) -> int:
        return -(-num_tokens // self.page_size)

    def pages_needed(self, request, total_tokens: int) -> List[int]:
        """New pages each group needs to hold ``total_tokens`` of the request
        (servelab/kv_cache/manager.py:74-76)."""
        want = self.pages_for(total_tokens)
        return [max(0, want - len(g.tables[request])) for g in self.page_groups]

    def can_ever_hold(self, total_tokens: int) -> bool:
        """False when a request of this length exceeds a whole pool
        (servelab/engine/scheduler.py:211-215)."""
        return self.pages_for(total_tokens) <= self.num_pages

    def can_admit(self, total_tokens: int) -> bool:
        """Whether a request that is not open yet could be opened and grown to
        ``total_tokens`` right now (a state slot and the pages of every group
        are free).  Takes nothing."""
        need = self.pages_for(total_tokens)
        return self.state_slots.num_free > 0 and \
            all(need <= g.allocator.num_free for g in self.page_groups)

    def grow(self, request, total_tokens: int) -> bool:
        """Make room for tokens [0, total_tokens) in every group; all groups or
        none.  Already held pages are kept, so growing twice is harmless
        (servelab/kv_cache/manager.py:153-191)."""
        need = self.pages_needed(request, total_tokens)
        for g, n in zip(self.page_groups, need):
            if n > g.allocator.num_free:
                g.allocator.alloc_fails += 1
                return False
        for g, n in zip(self.page_groups, need):
            if n:
                g.tables[request].extend(g.allocator.take(n))
        return True

    def commit(self, request, total_tokens: int) -> None:
        """Tokens [0, total_tokens) are now cached.  Window groups give back
        the pages that no later query can see: a query at p >= total sees keys
        r > p - W, so a page whose last token is <= total - W is dead."""
        self.lengths[request] = total_tokens
        bs = self.page_size
        for g in self.page_groups:
            if g.window is None:
                continue
            table = g.tables[request]
            dead_pages = max(0, (total_tokens - g.window + 1) // bs)
            for j in range(min(dead_pages, len(table))):
                if table[j] != RELEASED:
                    g.allocator.give([table[j]])
                    table[j] = RELEASED

    # ------------------------------------------------------------ queries
    def block_table(self, group: int, request) -> List[int]:
        return self.page_groups[group].tables[request]

    def slot(self, group: int, request, token_index: int) -> int:
        """Flat row of a token: table[i // bs] * bs + i % bs
        (servelab/kv_cache/manager.py:309-313)."""
        page = self.page_groups[group].tables[request][token_index // self.page_size]
        if page == RELEASED:
            raise AssertionError(f"token {token_index} of {request!r} lies in a released page")
        return page * self.page_size + token_index % self.page_size

    def state_slot(self, request) -> int:
        return self.state_slots.slot_of(request)

    def num_free_pages(self) -> int:
        """Free pages of the tightest group."""
        return min((g.allocator.num_free for g in self.page_groups), default=self.num_pages)

    def usage(self) -> float:
        used = max((g.allocator.num_used for g in self.page_groups), default=0)
        return used / self.num_pages

    def stats(self) -> dict:
        return {
            "pages_in_use": [g.allocator.num_used for g in self.page_groups],
            "high_water": [g.allocator.high_water for g in self.page_groups],
            "alloc_fails": sum(g.allocator.alloc_fails for g in self.page_groups),
            "state_slots_in_use": self.state_slots.num_slots - self.state_slots.num_free,
        }

    def check(self) -> None:
        """Every page is free or in exactly one table; every slot likewise."""
        for gi, g in enumerate(self.page_groups):
            seen = set()
            for request, table in g.tables.items():
                for p in table:
                    if p == RELEASED:
                        continue
                    if p in seen:
                        raise AssertionError(f"group {gi}: page {p} is in two tables")
                    if not g.allocator.is_held(p):
                        raise AssertionError(f"group {gi}: page {p} of {request!r} is on the free list")
                    seen.add(p)
            if len(seen) != g.allocator.num_used:
                raise AssertionError(
                    f"group {gi}: {g.allocator.num_used} pages held, {len(seen)} in tables")
            if set(g.tables) != set(self.lengths):
                raise AssertionError(f"group {gi}: tables and open requests differ")
        if set(self.state_slots.owners()) != set(self.lengths):
            raise AssertionError("state slots and open requests differ")
