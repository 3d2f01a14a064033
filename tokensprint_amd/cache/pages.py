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

from collections import OrderedDict
from dataclasses import dataclass, field

import numpy as np
import xxhash


class OutOfPages(RuntimeError):
    """A group's pool has fewer free pages than the request needs."""


class OutOfSlots(RuntimeError):
    """Every per-request state slot is taken."""


class PagePool:
    """Fixed pool of page ids: a FIFO free list and a reference count per page.

    A page is held by one request, or by several that share a cached prefix.  A free page
    may still carry the hash of the block it held (`tag`), so that a later request with the
    same prefix can take exactly that page back; the tag is dropped when the page is handed
    out for something else (`on_evict` tells the prefix index)."""

    def __init__(self, num_pages: int) -> None:
        if num_pages < 1:
            raise ValueError(f"a pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self.free: OrderedDict[int, None] = OrderedDict((i, None) for i in range(num_pages))
        self.refs: list[int] = [0] * num_pages
        self.tag: list[int | None] = [None] * num_pages
        self.on_evict = None               # callable(page, tag)

    @property
    def num_free(self) -> int:
        return len(self.free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self.free)

    def _evict_tag(self, page: int) -> None:
        if self.tag[page] is not None:
            if self.on_evict is not None:
                self.on_evict(page, self.tag[page])
            self.tag[page] = None

    def take(self) -> int:
        """The oldest free page, for new contents."""
        if not self.free:
            raise OutOfPages("no free page")
        page, _ = self.free.popitem(last=False)
        if self.refs[page] != 0:
            raise RuntimeError(f"page {page} is on the free list with {self.refs[page]} holders")
        self._evict_tag(page)
        self.refs[page] = 1
        return page

    def take_tagged(self, page: int) -> None:
        """Take a particular page for its contents: off the free list if nobody holds it,
        one more holder otherwise."""
        if self.refs[page] == 0:
            if page not in self.free:
                raise RuntimeError(f"page {page} has no holder and is not free")
            del self.free[page]
        self.refs[page] += 1

    def give_back(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise RuntimeError(f"page id {page} out of range")
        if self.refs[page] <= 0:
            raise RuntimeError(f"page {page} freed twice")
        self.refs[page] -= 1
        if self.refs[page] == 0:
            self.free[page] = None         # to the right end: reused last, so a cached
                                           # prefix survives as long as possible

    def check(self) -> None:
        """No page lost, none held and free at once."""
        for page in range(self.num_pages):
            if (self.refs[page] == 0) != (page in self.free):
                raise RuntimeError(f"page {page}: free list and holder count disagree")
            if self.refs[page] < 0:
                raise RuntimeError(f"page {page}: negative holder count")


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
    hashes: list[int] = field(default_factory=list)     # chained hash of every registered full page


class CacheManager:
    def __init__(self, groups: list[GroupLayout], page_size: int, num_pages,
                 num_slots: int, state_runs: tuple[int, ...] = ()) -> None:
        """`num_pages`: one int for every group, or a list with one int per group.
        `state_runs`: the runs that keep fixed-size state in the request's slot."""
        if page_size < 1:
            raise ValueError(f"page size must be >= 1, got {page_size}")
        self.groups = list(groups)
        self.state_runs = tuple(state_runs)
        self.page_size = page_size
        counts = [num_pages] * len(groups) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(groups):
            raise ValueError("one page count per group is needed")
        self.pools = [PagePool(n) for n in counts]
        self.slots = StateSlots(num_slots)
        self.live: dict[object, RequestCache] = {}
        # prefix cache (off until enabled): hash of a full page -> its page id in every group
        self.prefix_index: dict[int, tuple[int, ...]] | None = None
        self.prefix_tokens: dict[int, tuple[int, ...]] = {}   # the same keys: a page's tokens

    # ------------------------------------------------------------ prefix cache
    # The reference keeps a chained xxh64 per full block, a hash -> block map, blocks that
    # keep their hash while free, reference counts for sharing, and never takes the last
    # block of a request from the cache (engine/generation/block_manager.py:72-93,161-211,
    # 406-475).  The same here, over all groups at once; only for models whose groups all
    # keep every key (a window group gives pages back, so its prefix is not there to share)
    # and that keep nothing else per request: state in a slot is what the whole prefix
    # made of it, and no page holds a copy to start from.
    def enable_prefix_cache(self) -> None:
        if any(g.window is not None for g in self.groups):
            raise ValueError("prefix caching needs every cache group to keep all keys")
        if self.state_runs:
            raise ValueError(
                f"prefix caching cannot serve runs {list(self.state_runs)}, which keep "
                "fixed-size state per request: a request that starts behind cached pages "
                "would start with empty state")
        if self.prefix_index is None:
            self.prefix_index = {}
            for g, pool in enumerate(self.pools):
                pool.on_evict = lambda page, tag, g=g: self._evicted(g, page, tag)

    def _evicted(self, g: int, page: int, tag: int) -> None:
        entry = self.prefix_index.get(tag)
        if entry is not None and entry[g] == page:
            # one group's page is gone: the block is no longer whole
            del self.prefix_index[tag]
            self.prefix_tokens.pop(tag, None)
            for g2, page2 in enumerate(entry):
                if g2 != g and self.pools[g2].tag[page2] == tag:
                    self.pools[g2].tag[page2] = None

    @staticmethod
    def block_hash(token_ids, prefix: int = -1) -> int:
        """64-bit hash of a block of token ids chained to the hash of the blocks before."""
        h = xxhash.xxh64()
        if prefix != -1:
            h.update(prefix.to_bytes(8, "little"))
        h.update(np.asarray(token_ids, dtype=np.int64).tobytes())
        return h.intdigest()

    def match_prefix(self, token_ids) -> list[tuple[int, tuple[int, ...]]]:
        """(hash, pages) of the leading full pages of `token_ids` that are cached, never
        including the page that holds the last token."""
        if self.prefix_index is None:
            return []
        P, out, h = self.page_size, [], -1
        for i in range((len(token_ids) - 1) // P):
            h = self.block_hash(token_ids[i * P:(i + 1) * P], h)
            pages = self.prefix_index.get(h)
            # a hit counts only with equal tokens (two blocks may share a hash), and the
            # first miss ends the prefix whatever later blocks would match
            if pages is None or self.prefix_tokens[h] != tuple(token_ids[i * P:(i + 1) * P]):
                break
            out.append((h, pages))
        return out

    def register_full_pages(self, rc: RequestCache, token_ids, computed: int) -> None:
        """Make the pages of `rc` that are full and computed (positions < `computed`)
        findable by their contents."""
        if self.prefix_index is None:
            return
        P = self.page_size
        full = min(computed, len(token_ids)) // P
        while len(rc.hashes) < full:
            i = len(rc.hashes)
            h = self.block_hash(token_ids[i * P:(i + 1) * P], rc.hashes[-1] if rc.hashes else -1)
            rc.hashes.append(h)
            if h not in self.prefix_index:
                pages = tuple(table[i] for table in rc.tables)
                self.prefix_index[h] = pages
                self.prefix_tokens[h] = tuple(token_ids[i * P:(i + 1) * P])
                for g, page in enumerate(pages):
                    self.pools[g].tag[page] = h

    # ------------------------------------------------------------ admission
    def admit(self, request_id, token_ids=None) -> RequestCache:
        """A slot and empty block tables; with `token_ids` and the prefix cache enabled,
        tables that already hold the request's cached prefix (rc.num_tokens tells how far)."""
        if request_id in self.live:
            raise RuntimeError(f"request {request_id!r} is already live")
        slot = self.slots.take(request_id)
        rc = RequestCache(request_id, slot, [[] for _ in self.groups],
                          released=[0] * len(self.groups))
        self.live[request_id] = rc
        if token_ids is not None:
            for h, pages in self.match_prefix(token_ids):
                for g, page in enumerate(pages):
                    self.pools[g].take_tagged(page)
                    rc.tables[g].append(page)
                rc.hashes.append(h)
            rc.num_tokens = len(rc.hashes) * self.page_size
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

    def can_extend_all(self, wanted: list[tuple[RequestCache, int]]) -> bool:
        """True if every (request, new length) of `wanted` can be extended, one after the
        other in any order (pages a window lets go on the way are not counted on)."""
        need = [0] * len(self.pools)
        for rc, new_len in wanted:
            if self._fits_as_is(rc, new_len):
                continue
            for g, n in enumerate(self.pages_needed(rc, new_len)):
                need[g] += max(n, 0)
        return all(n <= pool.num_free for n, pool in zip(need, self.pools))

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
                table.append(self.pools[g].take())
        rc.num_tokens = new_len

    def shrink(self, rc: RequestCache, new_len: int) -> None:
        """Undo an `extend` whose tokens will not be computed after all: the request holds
        `new_len` tokens again and the pages beyond them go back.  (Pages a window let go
        on the way stay gone: no query from `new_len` on could see them.)"""
        if new_len > rc.num_tokens:
            raise ValueError(f"cannot shrink a request from {rc.num_tokens} to {new_len}")
        if new_len < len(rc.hashes) * self.page_size:
            raise ValueError("cannot shrink a request into its registered pages")
        total = -(-new_len // self.page_size)
        for g, table in enumerate(rc.tables):
            while len(table) > max(total, rc.released[g]):
                page = table.pop()
                if page >= 0:
                    self.pools[g].give_back(page)
        rc.num_tokens = new_len

    def release_passed(self, rc: RequestCache) -> None:
        """Give back the pages no query at position >= rc.num_tokens can see."""
        for g, table in enumerate(rc.tables):
            keep_from = min(self._first_kept_page(g, rc.num_tokens), len(table))
            for i in range(rc.released[g], keep_from):
                if table[i] >= 0:
                    self.pools[g].give_back(table[i])
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
                    self.pools[g].give_back(page)
            table.clear()
            rc.released[g] = 0
        self.slots.give_back(rc.slot, rc.request_id)
        rc.hashes.clear()
        rc.num_tokens = 0
        del self.live[rc.request_id]

    # ------------------------------------------------------------ checks
    def check(self) -> None:
        """Every page's holder count equals the live tables that name it; slots likewise."""
        for g, pool in enumerate(self.pools):
            pool.check()
            holders = [0] * pool.num_pages
            for rc in self.live.values():
                seen = set()
                for page in rc.tables[g]:
                    if page < 0:
                        continue
                    if page in seen:
                        raise RuntimeError(f"page {page} of group {g} twice in one table")
                    seen.add(page)
                    holders[page] += 1
            if holders != pool.refs:
                bad = next(i for i in range(pool.num_pages) if holders[i] != pool.refs[i])
                raise RuntimeError(f"group {g} page {bad}: {pool.refs[bad]} holders counted, "
                                   f"{holders[bad]} tables name it")
            if self.prefix_index is None and max(holders, default=0) > 1:
                raise RuntimeError(f"group {g}: a page is shared without a prefix cache")
        if self.prefix_index is not None:
            for h, pages in self.prefix_index.items():
                for g, page in enumerate(pages):
                    if self.pools[g].tag[page] != h:
                        raise RuntimeError(f"prefix index names page {page} of group {g} "
                                           "whose tag differs")
        slots = [rc.slot for rc in self.live.values()]
        if len(set(slots)) != len(slots):
            raise RuntimeError("a state slot is held twice")
        if self.slots.num_free + len(slots) != self.slots.num_slots:
            raise RuntimeError("a state slot is lost")
