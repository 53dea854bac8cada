"""Host side of the cache: pages, block tables and per-request state slots.  Device-free.

Keys and values live in pages of ``page_size`` positions.  Layers with the same needs form
a *group* (all keys, or a window of them); each group has a page pool and one block table
row per request slot: ``table[slot, i]`` is the page holding positions
``[i * page_size, (i + 1) * page_size)`` of the request in that slot, or the null page 0.
Pages come back when a request ends and, in a windowed group, as soon as the window has
moved past them; returned pages are handed out again first.

The reference splits this over ``BlockPool`` (rapid_llm/engine/block_pool.py: null block 0
at :19-22,:190-192, all-or-nothing ``get_new_blocks`` :234), ``KVCacheCoordinator``
(rapid_llm/engine/kv_cache_spec.py: groups :480-549, tail-first free :595-606,
``remove_skipped_blocks`` for windows :608-634) and per-request slots
(rapid_llm/engine/batch_planner.py:112,:1033-1035).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

NULL_PAGE = 0


class CacheError(RuntimeError):
    pass


class PagePool:
    """``num_pages`` physical pages; page 0 is the null page and is never handed out."""

    def __init__(self, num_pages: int) -> None:
        if num_pages < 2:
            raise CacheError(f"a page pool needs at least 2 pages (page 0 is null), got {num_pages}")
        self.num_pages = num_pages
        # stack: the page freed last is taken first; initially 1, 2, 3, ... in order
        self._free: list[int] = list(range(num_pages - 1, 0, -1))
        self._held = np.zeros(num_pages, dtype=bool)

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_usable(self) -> int:
        return self.num_pages - 1

    def take(self, count: int) -> list[int] | None:
        """``count`` pages, or ``None`` with nothing taken when fewer are free."""
        if count < 0:
            raise CacheError(f"cannot take {count} pages")
        if count > len(self._free):
            return None
        pages = [self._free.pop() for _ in range(count)]
        self._held[pages] = True
        return pages

    def give_back(self, pages) -> None:
        for page in pages:
            page = int(page)
            if page == NULL_PAGE:
                raise CacheError("the null page cannot be given back")
            if not 0 < page < self.num_pages:
                raise CacheError(f"page {page} is not in this pool of {self.num_pages}")
            if not self._held[page]:
                raise CacheError(f"page {page} is given back twice")
            self._held[page] = False
            self._free.append(page)

    def held(self) -> list[int]:
        return [int(p) for p in np.nonzero(self._held)[0]]


@dataclass(frozen=True)
class GroupSpec:
    """Layers that share page ids.  ``window`` 0: every position is kept."""

    group_id: int
    window: int
    layers: tuple[int, ...]


@dataclass
class _Request:
    request_id: str
    slot: int
    reserved: int = 0  # positions [0, reserved) are addressable in every group
    capacity: int = 0  # positions the mapped pages reach to (reserved rounded up to whole pages)
    trimmed: list[int] = field(default_factory=list)  # per group: pages below this index were returned


class CacheManager:
    """Slots, pages and block tables for up to ``max_seqs`` live requests."""

    def __init__(
        self,
        groups: list[GroupSpec],
        num_pages: int | dict[int, int],
        page_size: int,
        max_seqs: int,
        max_seq_len: int,
    ) -> None:
        if page_size < 1:
            raise CacheError(f"page_size must be positive, got {page_size}")
        if max_seqs < 1:
            raise CacheError(f"max_seqs must be positive, got {max_seqs}")
        self.groups = list(groups)
        self.page_size = page_size
        self.max_seqs = max_seqs
        self.max_seq_len = max_seq_len
        self.max_pages_per_seq = max(1, -(-max_seq_len // page_size))
        self.pools: dict[int, PagePool] = {}
        self.tables: dict[int, np.ndarray] = {}
        for g in self.groups:
            n = num_pages[g.group_id] if isinstance(num_pages, dict) else num_pages
            self.pools[g.group_id] = PagePool(n)
            self.tables[g.group_id] = np.zeros((max_seqs, self.max_pages_per_seq), dtype=np.int32)
        self._free_slots: list[int] = list(range(max_seqs - 1, -1, -1))
        self._requests: dict[str, _Request] = {}
        # slots whose table rows changed since the device copy was last refreshed
        self.dirty_slots: set[int] = set()
        # slots taken since the device state was last cleared
        self.fresh_slots: set[int] = set()

    # ------------------------------------------------------------------ slots
    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def has(self, request_id: str) -> bool:
        return request_id in self._requests

    def slot_of(self, request_id: str) -> int:
        return self._requests[request_id].slot

    def reserved(self, request_id: str) -> int:
        return self._requests[request_id].reserved

    def live_requests(self) -> list[str]:
        return list(self._requests)

    def admit(self, request_id: str) -> int | None:
        """Give the request a slot (its block-table row and state); ``None`` if none is free."""
        if request_id in self._requests:
            raise CacheError(f"request {request_id!r} is already admitted")
        if not self._free_slots:
            return None
        slot = self._free_slots.pop()
        self._requests[request_id] = _Request(request_id, slot, trimmed=[0] * len(self.groups))
        self.fresh_slots.add(slot)
        return slot

    # ------------------------------------------------------------------ pages
    def _first_needed_page(self, group: GroupSpec, next_position: int) -> int:
        """Index of the first page a query at ``next_position`` or later can still read."""
        if group.window <= 0:
            return 0
        first_pos = max(0, next_position - group.window + 1)
        return first_pos // self.page_size

    def pages_needed(self, request_id: str, upto: int, start: int | None = None) -> dict[int, int]:
        """New pages per group that ``reserve(request_id, upto, start)`` would take."""
        req = self._requests[request_id]
        if start is None:
            start = req.reserved
        need = {}
        last = -(-upto // self.page_size)  # pages [0, last) must be addressable
        for gi, g in enumerate(self.groups):
            first = max(req.trimmed[gi], self._first_needed_page(g, start))
            row = self.tables[g.group_id][req.slot]
            need[g.group_id] = int(np.count_nonzero(row[first:last] == NULL_PAGE)) if last > first else 0
        return need

    def reserve(self, request_id: str, upto: int, start: int | None = None) -> bool:
        """Make positions ``[start, upto)`` writable and everything a query in that span reads
        addressable, in every group.  All or nothing: ``False`` leaves pools and tables as
        they were (rapid_llm/engine/kv_cache_spec.py:526-549).  ``start`` defaults to what
        is reserved already."""
        req = self._requests[request_id]
        if upto > self.max_seq_len:
            raise CacheError(
                f"request {request_id!r} asks for {upto} positions; the cache is laid out for "
                f"sequences of at most {self.max_seq_len}"
            )
        if upto <= req.capacity:
            # the pages that were mapped last reach that far (a decoded token needs a new page
            # only every page_size-th step); pages a window has passed stay returned
            req.reserved = max(req.reserved, upto)
            return True
        if start is None:
            start = req.reserved
        need = self.pages_needed(request_id, upto, start)
        for gid, count in need.items():
            if count > self.pools[gid].num_free:
                return False
        last = -(-upto // self.page_size)
        for gi, g in enumerate(self.groups):
            if need[g.group_id] == 0:
                continue
            first = max(req.trimmed[gi], self._first_needed_page(g, start))
            row = self.tables[g.group_id][req.slot]
            holes = [i for i in range(first, last) if row[i] == NULL_PAGE]
            pages = self.pools[g.group_id].take(len(holes))
            assert pages is not None
            for i, page in zip(holes, pages):
                row[i] = page
            self.dirty_slots.add(req.slot)
        req.reserved = max(req.reserved, upto)
        req.capacity = max(req.capacity, last * self.page_size)
        return True

    def trim(self, request_id: str, next_position: int) -> int:
        """Give back the pages of windowed groups that no query at ``next_position`` or later
        can read; their table entries become the null page.  Returns the number returned."""
        req = self._requests[request_id]
        returned = 0
        for gi, g in enumerate(self.groups):
            first = self._first_needed_page(g, next_position)
            if first <= req.trimmed[gi]:
                continue
            row = self.tables[g.group_id][req.slot]
            pages = [int(p) for p in row[req.trimmed[gi] : first] if p != NULL_PAGE]
            if pages:
                self.pools[g.group_id].give_back(pages)
                row[req.trimmed[gi] : first] = NULL_PAGE
                self.dirty_slots.add(req.slot)
                returned += len(pages)
            req.trimmed[gi] = first
        return returned

    def release(self, request_id: str) -> None:
        """The request is over: every page and the slot come back, tail first
        (rapid_llm/engine/kv_cache_spec.py:595-606)."""
        req = self._requests.pop(request_id, None)
        if req is None:
            raise CacheError(f"request {request_id!r} holds nothing (released twice?)")
        for g in self.groups:
            row = self.tables[g.group_id][req.slot]
            pages = [int(p) for p in row[::-1] if p != NULL_PAGE]
            if pages:
                self.pools[g.group_id].give_back(pages)
            row[:] = NULL_PAGE
        self.dirty_slots.add(req.slot)
        self._free_slots.append(req.slot)

    # ------------------------------------------------------------------ views
    def pages_of(self, request_id: str, group_id: int) -> list[int]:
        row = self.tables[group_id][self._requests[request_id].slot]
        return [int(p) for p in row if p != NULL_PAGE]

    def num_free_pages(self, group_id: int | None = None) -> int:
        if group_id is not None:
            return self.pools[group_id].num_free
        # a model without paged layers is never short of pages
        return min((p.num_free for p in self.pools.values()), default=1 << 30)

    def capacity_tokens(self) -> int:
        """Positions one request can hold at most if it has the pool to itself."""
        usable = min((p.num_usable for p in self.pools.values()), default=None)
        return self.max_seq_len if usable is None else usable * self.page_size

    def check_invariants(self) -> None:
        """No page lost, none held twice: every held page sits in exactly one table cell."""
        for g in self.groups:
            pool = self.pools[g.group_id]
            table = self.tables[g.group_id]
            used = table[table != NULL_PAGE]
            if len(used) != len(set(used.tolist())):
                raise CacheError(f"group {g.group_id}: a page appears in two table cells")
            if sorted(used.tolist()) != pool.held():
                raise CacheError(f"group {g.group_id}: held pages and table cells disagree")
            if pool.num_free + len(used) != pool.num_usable:
                raise CacheError(f"group {g.group_id}: pages were lost")
            live = {r.slot for r in self._requests.values()}
            for slot in range(self.max_seqs):
                if slot not in live and np.any(table[slot] != NULL_PAGE):
                    raise CacheError(f"group {g.group_id}: free slot {slot} still maps pages")
        live = [r.slot for r in self._requests.values()]
        if len(live) != len(set(live)) or set(live) & set(self._free_slots):
            raise CacheError("a slot is held twice")
        if len(live) + len(self._free_slots) != self.max_seqs:
            raise CacheError("a slot was lost")
