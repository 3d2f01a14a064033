"""Host bookkeeping of the paged cache: pools, groups, block tables, state slots.

What the reference's BlockManager keeps (engine/generation/block_manager.py:38-70,
123-159,270-322): a fixed pool of pages, a FIFO free list (taken from the left, given
back on the right), a used set, and a per-request block table from logical to physical
page.  Added here: several groups of layers, each with a pool and per-request table of
its own, so that layers that see every earlier key and layers that see only a window of
them are accounted separately; a window group gives pages back as soon as no later query
can see them; and fixed-size state slots, one per live request.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field


class OutOfPages(RuntimeError):
    """A group's pool has fewer free pages than the request needs."""


class OutOfSlots(RuntimeError):
    """Every per-request state slot is taken."""


class PagePool:
    """Fixed pool of page ids with a FIFO free list and an owner per page."""

    def __init__(self, num_pages: int) -> None:
        if num_pages < 1:
            raise ValueError(f"a pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self.free: deque[int] = deque(range(num_pages))
        self.owner: list[object | None] = [None] * num_pages   # None = free

    @property
    def num_free(self) -> int:
        return len(self.free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self.free)

    def take(self, owner) -> int:
        if owner is None:
            raise ValueError("a page needs an owner")
        if not self.free:
            raise OutOfPages("no free page")
        page = self.free.popleft()
        if self.owner[page] is not None:
            raise RuntimeError(f"page {page} is on the free list but owned by {self.owner[page]}")
        self.owner[page] = owner
        return page

    def give_back(self, page: int, owner) -> None:
        if not 0 <= page < self.num_pages:
            raise RuntimeError(f"page id {page} out of range")
        if self.owner[page] is None:
            raise RuntimeError(f"page {page} freed twice")
        if self.owner[page] != owner:
            raise RuntimeError(f"page {page} is owned by {self.owner[page]}, not {owner}")
        self.owner[page] = None
        self.free.append(page)

    def check(self) -> None:
        """No page lost, none held and free at once, none on the free list twice."""
        free = list(self.free)
        if len(set(free)) != len(free):
            raise RuntimeError("a page is on the free list twice")
        for page in range(self.num_pages):
            if (self.owner[page] is None) != (page in set(free)):
                raise RuntimeError(f"page {page}: free list and owner disagree")


class StateSlots:
    """Slot ids for fixed-size per-request state; lowest free id first."""

    def __init__(self, num_slots: int) -> None:
        if num_slots < 1:
            raise ValueError("need at least one state slot")
        self.num_slots = num_slots
        self.free: list[int] = list(range(num_slots - 1, -1, -1))
        self.owner: list[object | None] = [None] * num_slots

    @property
    def num_free(self) -> int:
        return len(self.free)

    def take(self, owner) -> int:
        if not self.free:
            raise OutOfSlots(f"all {self.num_slots} state slots are in use")
        slot = self.free.pop()
        self.owner[slot] = owner
        return slot

    def give_back(self, slot: int, owner) -> None:
        if self.owner[slot] is None:
            raise RuntimeError(f"slot {slot} freed twice")
        if self.owner[slot] != owner:
            raise RuntimeError(f"slot {slot} is owned by {self.owner[slot]}, not {owner}")
        self.owner[slot] = None
        self.free.append(slot)
        self.free.sort(reverse=True)


@dataclass(frozen=True)
class GroupLayout:
    """One group of runs whose caches share page ids.

    `window` None: every earlier key stays; W: a query at position p sees keys
    p-W+1..p, so a page whose last position is below that for every coming query
    is given back.
    """

    num_kv_heads: int
    head_dim: int
    window: int | None
    runs: tuple[int, ...]          # run indices whose caches live in this group


@dataclass
class RequestCache:
    """What one live request holds: a state slot and a block table per group."""

    request_id: object
    slot: int
    tables: list[list[int]]        # per group: logical page -> physical id, -1 = given back
    num_tokens: int = 0            # positions [0, num_tokens) are in the cache
    released: list[int] = field(default_factory=list)   # per group: leading pages given back


class CacheManager:
    def __init__(self, groups: list[GroupLayout], page_size: int, num_pages,
                 num_slots: int) -> None:
        """`num_pages`: one int for every group, or a list with one int per group."""
        if page_size < 1:
            raise ValueError(f"page size must be >= 1, got {page_size}")
        self.groups = list(groups)
        self.page_size = page_size
        counts = [num_pages] * len(groups) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(groups):
            raise ValueError("one page count per group is needed")
        self.pools = [PagePool(n) for n in counts]
        self.slots = StateSlots(num_slots)
        self.live: dict[object, RequestCache] = {}

    # ------------------------------------------------------------ admission
    def admit(self, request_id) -> RequestCache:
        if request_id in self.live:
            raise RuntimeError(f"request {request_id!r} is already live")
        slot = self.slots.take(request_id)
        rc = RequestCache(request_id, slot, [[] for _ in self.groups],
                          released=[0] * len(self.groups))
        self.live[request_id] = rc
        return rc

    # ------------------------------------------------------------ growth
    def _first_kept_page(self, g: int, first_query_pos: int) -> int:
        """Index of the first page a query at `first_query_pos` (or later) can see."""
        window = self.groups[g].window
        if window is None:
            return 0
        return max(0, first_query_pos - window + 1) // self.page_size

    def pages_needed(self, rc: RequestCache, new_len: int) -> list[int]:
        """Per group, free pages that extending to `new_len` tokens takes from the
        pool, counting the pages the window lets go first."""
        P = self.page_size
        total = -(-new_len // P)
        out = []
        for g, table in enumerate(rc.tables):
            released_now = sum(1 for i in range(rc.released[g],
                                                min(self._first_kept_page(g, rc.num_tokens),
                                                    len(table))) if table[i] >= 0)
            out.append(max(0, total - len(table)) - released_now)
        return out

    def _fits_as_is(self, rc: RequestCache, new_len: int) -> bool:
        """True if no group has to take or give back a page for `new_len` tokens: the
        common decode step, kept cheap."""
        P = self.page_size
        for g, table in enumerate(rc.tables):
            if len(table) * P < new_len:
                return False
            if self.groups[g].window is not None and \
                    self._first_kept_page(g, rc.num_tokens) > rc.released[g]:
                return False
        return True

    def can_extend(self, rc: RequestCache, new_len: int) -> bool:
        if self._fits_as_is(rc, new_len):
            return True
        return all(need <= pool.num_free
                   for need, pool in zip(self.pages_needed(rc, new_len), self.pools))

    def extend(self, rc: RequestCache, new_len: int) -> None:
        """Make positions [rc.num_tokens, new_len) writable; all groups or none."""
        if new_len < rc.num_tokens:
            raise ValueError(f"cannot shrink a request from {rc.num_tokens} to {new_len}")
        if self._fits_as_is(rc, new_len):
            rc.num_tokens = new_len
            return
        if not self.can_extend(rc, new_len):
            raise OutOfPages(
                f"request {rc.request_id!r} needs {self.pages_needed(rc, new_len)} pages "
                f"per group, free are {[p.num_free for p in self.pools]}")
        self.release_passed(rc)
        total = -(-new_len // self.page_size)
        for g, table in enumerate(rc.tables):
            while len(table) < total:
                table.append(self.pools[g].take(rc.request_id))
        rc.num_tokens = new_len

    def release_passed(self, rc: RequestCache) -> None:
        """Give back the pages no query at position >= rc.num_tokens can see."""
        for g, table in enumerate(rc.tables):
            keep_from = min(self._first_kept_page(g, rc.num_tokens), len(table))
            for i in range(rc.released[g], keep_from):
                if table[i] >= 0:
                    self.pools[g].give_back(table[i], rc.request_id)
                    table[i] = -1
            rc.released[g] = max(rc.released[g], keep_from)

    # ------------------------------------------------------------ release
    def free(self, rc: RequestCache) -> None:
        """Everything the request holds goes back (finish or preemption).
        Pages return in reverse table order, as block_manager.py:282-285 does."""
        if self.live.get(rc.request_id) is not rc:
            raise RuntimeError(f"request {rc.request_id!r} is not live")
        for g, table in enumerate(rc.tables):
            for page in reversed(table):
                if page >= 0:
                    self.pools[g].give_back(page, rc.request_id)
            table.clear()
            rc.released[g] = 0
        self.slots.give_back(rc.slot, rc.request_id)
        rc.num_tokens = 0
        del self.live[rc.request_id]

    # ------------------------------------------------------------ checks
    def check(self) -> None:
        """Every used page is in exactly one live table; slots likewise."""
        for g, pool in enumerate(self.pools):
            pool.check()
            seen: dict[int, object] = {}
            for rc in self.live.values():
                for page in rc.tables[g]:
                    if page < 0:
                        continue
                    if page in seen:
                        raise RuntimeError(f"page {page} of group {g} is in two tables")
                    seen[page] = rc.request_id
                    if pool.owner[page] != rc.request_id:
                        raise RuntimeError(f"page {page} of group {g}: owner mismatch")
            if len(seen) != pool.num_used:
                raise RuntimeError(f"group {g}: {pool.num_used} pages used, {len(seen)} in tables")
        slots = [rc.slot for rc in self.live.values()]
        if len(set(slots)) != len(slots):
            raise RuntimeError("a state slot is held twice")
        if self.slots.num_free + len(slots) != self.slots.num_slots:
            raise RuntimeError("a state slot is lost")
