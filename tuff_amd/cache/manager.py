"""Book-keeping of the cache, without tensors: which pages and which state slot each live
request holds.

Cache entries that grow a token at a time (PagedKV) are sorted into groups by what they need
to keep: all positions, or a window of the last W.  A group has a page pool and, per request,
a block table of its own; all entries of a group share the page numbering.  Entries of fixed
size (FixedState) live in one slot per request.  Pages go back to their pool when the request
ends or when a window has moved past them, and are handed out again (last freed, first used).

The reference has nothing of this: one request, one contiguous window sized at start
(src/lfm25_engine.c:53-60).
"""
from __future__ import annotations

import dataclasses
from typing import Hashable, Optional

from ..parts.base import FixedState, PagedKV

FREED = -1


class CacheError(RuntimeError):
    """Misuse of the cache manager: a page freed twice, an unknown request, ..."""


class OutOfPages(CacheError):
    """A pool cannot supply the pages a step needs.  Nothing was taken."""


class OutOfSlots(CacheError):
    """Every state slot is held by a live request."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must be >= 0")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))      # pop() hands out page 0 first
        self._held = [False] * num_pages
        self.allocations = 0                                   # pages handed out so far, ever

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self, n: int) -> list[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} free of {self.num_pages}")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._held[p] = True
        self.allocations += n
        return pages

    def free(self, pages) -> None:
        for p in pages:
            if not (0 <= p < self.num_pages) or not self._held[p]:
                raise CacheError(f"page {p} is freed but not held")
            self._held[p] = False
            self._free.append(p)

    def is_held(self, p: int) -> bool:
        return self._held[p]


@dataclasses.dataclass
class CacheGroup:
    window: Optional[int]
    entries: list[int]            # cache entry ids in this group
    pool: PagePool


@dataclasses.dataclass
class CacheLayout:
    """Which cache entries exist and how they are grouped; derived from a model's run order."""
    paged: dict[int, PagedKV]                   # keyed by entry id: an int, or (int, j) for a mixer with several
    states: dict[int, FixedState]
    group_windows: list[Optional[int]]          # one per group
    group_of_entry: dict[int, int]

    @staticmethod
    def from_specs(specs: dict[int, object]) -> "CacheLayout":
        paged = {i: s for i, s in specs.items() if isinstance(s, PagedKV)}
        states = {i: s for i, s in specs.items() if isinstance(s, FixedState)}
        other = [s for s in specs.values() if s is not None and not isinstance(s, (PagedKV, FixedState))]
        if other:
            raise CacheError(f"unknown cache declaration {other[0]!r}")
        windows: list[Optional[int]] = []
        group_of = {}
        for i in sorted(paged, key=lambda e: e if isinstance(e, tuple) else (e, -1)):
            w = paged[i].window
            if w not in windows:
                windows.append(w)
            group_of[i] = windows.index(w)
        return CacheLayout(paged, states, windows, group_of)

    def bytes_per_token(self, elem_size: int) -> int:
        return sum(s.num_kv_heads * (s.head_dim + s.v_dim) * elem_size for s in self.paged.values())

    def state_bytes_per_request(self) -> int:
        return sum(s.nbytes() for s in self.states.values())


@dataclasses.dataclass
class _Request:
    slot: int
    length: int = 0
    tables: list = dataclasses.field(default_factory=list)     # per group: page id or FREED per block
    arrays: dict = dataclasses.field(default_factory=dict)     # per group: the table as int32 array, while current


class CacheManager:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages: int | list[int], num_slots: int):
        if page_size < 1:
            raise ValueError("page_size must be >= 1")
        self.layout, self.page_size, self.num_slots = layout, int(page_size), int(num_slots)
        n_groups = len(layout.group_windows)
        counts = [num_pages] * n_groups if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != n_groups:
            raise ValueError(f"{n_groups} cache groups but {len(counts)} pool sizes")
        self.groups = [CacheGroup(w, [e for e, g in layout.group_of_entry.items() if g == gi], PagePool(c))
                       for gi, (w, c) in enumerate(zip(layout.group_windows, counts))]
        self._free_slots = list(range(self.num_slots - 1, -1, -1))
        self._requests: dict[Hashable, _Request] = {}
        #: debugging aid: called as on_free(group index, pages) whenever pages go back to a pool
        self.on_free = None

    # ------------------------------------------------------------------ requests
    def __contains__(self, req_id) -> bool:
        return req_id in self._requests

    def live(self) -> list:
        return list(self._requests)

    def _req(self, req_id) -> _Request:
        r = self._requests.get(req_id)
        if r is None:
            raise CacheError(f"request {req_id!r} holds no cache")
        return r

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self, req_id) -> int:
        """Gives the request a state slot and empty block tables.  Returns the slot; its
        state must be zeroed by the owner of the tensors before the first step."""
        if req_id in self._requests:
            raise CacheError(f"request {req_id!r} is already live")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.num_slots} state slots are in use")
        slot = self._free_slots.pop()
        self._requests[req_id] = _Request(slot, 0, [[] for _ in self.groups])
        return slot

    def length(self, req_id) -> int:
        return self._req(req_id).length

    def slot(self, req_id) -> int:
        return self._req(req_id).slot

    # -------------------------------------------------------------------- pages
    def _first_needed_block(self, group: CacheGroup, length: int) -> int:
        """Blocks below this index hold only positions no later token of the request reads."""
        if group.window is None:
            return 0
        first_pos = max(0, length - group.window + 1)     # earliest key the next token reads
        return first_pos // self.page_size

    def pages_needed(self, req_id, n_new: int) -> list[int]:
        """Pages each group must still supply to hold n_new more tokens (after giving back
        what a window has passed)."""
        r = self._req(req_id)
        out = []
        for gi, g in enumerate(self.groups):
            have = len(r.tables[gi])
            want = -(-(r.length + n_new) // self.page_size)
            out.append(max(0, want - have))
        return out

    def reclaimable(self, req_id) -> list[int]:
        """Pages per group that extend() would give back before allocating."""
        r = self._req(req_id)
        out = []
        for gi, g in enumerate(self.groups):
            if g.window is None:
                out.append(0)
                continue
            lo = self._first_needed_block(g, r.length)
            out.append(sum(1 for p in r.tables[gi][:lo] if p != FREED))
        return out

    def can_extend(self, req_id, n_new: int) -> bool:
        need, back = self.pages_needed(req_id, n_new), self.reclaimable(req_id)
        return all(n <= g.pool.num_free + b for n, b, g in zip(need, back, self.groups))

    def extend(self, req_id, n_new: int) -> None:
        """Makes room for the next n_new tokens of the request in every group: first gives
        back pages a window has passed, then takes the new pages.  Raises OutOfPages and takes
        nothing if any pool is short."""
        if n_new < 0:
            raise ValueError("n_new must be >= 0")
        r = self._req(req_id)
        for gi, g in enumerate(self.groups):
            lo = self._first_needed_block(g, r.length)
            gone = [p for p in r.tables[gi][:lo] if p != FREED]
            if gone:
                r.arrays.pop(gi, None)
                self._give_back(gi, gone)
                for b in range(min(lo, len(r.tables[gi]))):
                    r.tables[gi][b] = FREED
        need = self.pages_needed(req_id, n_new)
        for n, g in zip(need, self.groups):
            if n > g.pool.num_free:
                raise OutOfPages(f"request {req_id!r}: {n} pages wanted, {g.pool.num_free} free "
                                 f"of {g.pool.num_pages} (window {g.window})")
        for gi, (n, g) in enumerate(zip(need, self.groups)):
            if n:
                r.arrays.pop(gi, None)
                r.tables[gi].extend(g.pool.alloc(n))
        r.length += n_new

    def _give_back(self, gi: int, pages: list) -> None:
        self.groups[gi].pool.free(pages)
        if pages and self.on_free is not None:
            self.on_free(gi, pages)

    def truncate(self, req_id, length: int) -> None:
        """Takes back an extend(): the request holds `length` tokens again.  Pages beyond are
        returned; pages a window freed meanwhile stay freed."""
        r = self._req(req_id)
        if length > r.length or length < 0:
            raise CacheError(f"cannot truncate request {req_id!r} from {r.length} to {length}")
        keep = -(-length // self.page_size)
        for gi, g in enumerate(self.groups):
            extra = [p for p in r.tables[gi][keep:] if p != FREED]
            self._give_back(gi, extra)
            del r.tables[gi][keep:]
        r.arrays.clear()
        r.length = length

    def release(self, req_id) -> None:
        """The request is over: all its pages and its slot are given back."""
        r = self._req(req_id)
        for gi, g in enumerate(self.groups):
            self._give_back(gi, [p for p in r.tables[gi] if p != FREED])
        self._free_slots.append(r.slot)
        del self._requests[req_id]

    # ------------------------------------------------------------------ lookups
    def block_table(self, req_id, group: int) -> list[int]:
        return self._req(req_id).tables[group]

    def block_table_array(self, req_id, group: int):
        """The block table as an int32 numpy array (kept until the table changes)."""
        import numpy as np
        r = self._req(req_id)
        a = r.arrays.get(group)
        if a is None:
            a = r.arrays[group] = np.asarray(r.tables[group], dtype=np.int32)
        return a

    def slot_of_position(self, req_id, group: int, pos: int) -> int:
        page = self._req(req_id).tables[group][pos // self.page_size]
        if page == FREED:
            raise CacheError(f"position {pos} of request {req_id!r} lies in a page that was given back")
        return page * self.page_size + pos % self.page_size

    def max_blocks(self) -> int:
        return max([len(t) for r in self._requests.values() for t in r.tables] + [1])

    # --------------------------------------------------------------- invariants
    def check(self) -> None:
        """Every page is free or held by exactly one block of one request; slots likewise."""
        for gi, g in enumerate(self.groups):
            owners: dict[int, tuple] = {}
            for rid, r in self._requests.items():
                for b, p in enumerate(r.tables[gi]):
                    if p == FREED:
                        continue
                    if p in owners:
                        raise CacheError(f"group {gi}: page {p} held twice: {owners[p]} and {(rid, b)}")
                    owners[p] = (rid, b)
                    if not g.pool.is_held(p):
                        raise CacheError(f"group {gi}: page {p} of {rid!r} is on the free list")
                want = -(-r.length // self.page_size)
                if len(r.tables[gi]) != want:
                    raise CacheError(f"group {gi}: request {rid!r} of length {r.length} has "
                                     f"{len(r.tables[gi])} blocks, expected {want}")
            if len(owners) + g.pool.num_free != g.pool.num_pages:
                raise CacheError(f"group {gi}: {len(owners)} held + {g.pool.num_free} free != "
                                 f"{g.pool.num_pages} pages (a page was lost)")
            if len(set(g.pool._free)) != len(g.pool._free):
                raise CacheError(f"group {gi}: a page is on the free list twice")
        slots = [r.slot for r in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise CacheError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.num_slots:
            raise CacheError("a state slot was lost")
