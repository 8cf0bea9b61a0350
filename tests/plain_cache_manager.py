"""The cache manager in plain Python: the oracle that the C++ cache manager of the host library is checked
against (same calls, same answers, same errors, under random orders of requests).

Host side of the cache: page pools, block tables and state slots. No tensors here.

The reference's BlockAllocator keeps a deque of reference-counted blocks and reuses the one
freed last (core/src/sched/block_manager.rs:14-58); BlockSpaceManager maps a sequence to its list
of blocks (:69-347), with one pool for all layers and a model-wide sliding window that wraps the
table (:129-135, :165-175). Here:

- Layers with equal needs form a *group* with a page pool and per-request block tables of its own;
  a group is either "full" (every key stays) or has a window W (only positions > p - W are read
  by a query at p).
- Pages are given back when a request ends, and, in a window group, as soon as the window has
  passed them. A freed page is the next one handed out (LIFO), so reuse is immediate.
- Beside the pages there are slots for per-request state of fixed size: one slot per live request,
  taken at its first tokens and given back with its pages.
- Nothing is shared between requests, so a page has one holder or none; giving back a page that is
  not held is an error (block_manager.rs:45-48 is the reference's double-free check).
"""
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence


class OutOfPages(RuntimeError):
    """A pool cannot supply the pages (or state slots) that an append needs."""


class CacheError(RuntimeError):
    """Misuse of the cache manager: unknown request, double free, a page held twice."""


class PagePool:
    """``num_pages`` page ids with a LIFO free list and a holder check."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must be >= 0")
        self.num_pages = int(num_pages)
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))   # page 0 is handed out first
        self._held = [False] * self.num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages("page pool of %d pages is exhausted" % self.num_pages)
        p = self._free.pop()
        if self._held[p]:
            raise CacheError("page %d was on the free list while held" % p)
        self._held[p] = True
        return p

    def release(self, page: int) -> None:
        if not (0 <= page < self.num_pages):
            raise CacheError("page %r does not exist" % (page,))
        if not self._held[page]:
            raise CacheError("page %d is given back twice" % page)
        self._held[page] = False
        self._free.append(page)

    def is_held(self, page: int) -> bool:
        return self._held[page]


@dataclass(frozen=True)
class GroupConfig:
    """One cache group: its page geometry and whether it keeps all keys or a window of them."""

    page_size: int
    num_pages: int
    window: Optional[int] = None


RELEASED = -1


@dataclass
class RequestCache:
    """What one live request holds."""

    request_id: Hashable
    state_slot: int
    num_tokens: int = 0                         # tokens whose keys and values are in the pages
    pending: int = 0                            # tokens appended but not yet committed (the running step's)
    tables: List[List[int]] = field(default_factory=list)     # per group: page of logical block i, or RELEASED
    first_live: List[int] = field(default_factory=list)       # per group: first block not yet released


class CacheManager:
    def __init__(self, groups: Sequence[GroupConfig], num_state_slots: int):
        for g in groups:
            if g.page_size <= 0:
                raise ValueError("page_size must be > 0")
            if g.window is not None and g.window <= 0:
                raise ValueError("window must be > 0 or None")
        self.groups = list(groups)
        self.pools = [PagePool(g.num_pages) for g in self.groups]
        self.num_state_slots = int(num_state_slots)
        self._free_slots: List[int] = list(range(self.num_state_slots - 1, -1, -1))
        self._requests: Dict[Hashable, RequestCache] = {}

    # ------------------------------------------------------------------ queries

    def has_request(self, rid: Hashable) -> bool:
        return rid in self._requests

    def request(self, rid: Hashable) -> RequestCache:
        try:
            return self._requests[rid]
        except KeyError:
            raise CacheError("request %r holds no cache" % (rid,))

    def live_requests(self) -> List[Hashable]:
        return list(self._requests)

    def num_free_pages(self, group: int = 0) -> int:
        return self.pools[group].num_free

    def num_free_state_slots(self) -> int:
        return len(self._free_slots)

    def num_tokens(self, rid: Hashable) -> int:
        return self.request(rid).num_tokens

    def pages_needed(self, rid: Optional[Hashable], n_new: int, held_tokens: Optional[int] = None) -> List[int]:
        """New pages per group that appending ``n_new`` tokens would take. ``rid`` None (or unknown)
        counts for a request that holds nothing yet."""
        out = []
        rc = self._requests.get(rid) if rid is not None else None
        for gi, g in enumerate(self.groups):
            have = len(rc.tables[gi]) if rc is not None else 0
            total = (rc.num_tokens + rc.pending if rc is not None else 0) + n_new
            out.append(max(0, -(-total // g.page_size) - have))
        return out

    def can_append(self, rid: Optional[Hashable], n_new: int, reserve_pages: int = 0) -> bool:
        """True if ``n_new`` more tokens of ``rid`` fit, leaving ``reserve_pages`` free in every group."""
        need = self.pages_needed(rid, n_new)
        if (rid is None or rid not in self._requests) and not self._free_slots:
            return False
        return all(self.pools[gi].num_free - need[gi] >= reserve_pages for gi in range(len(self.groups)))

    # ------------------------------------------------------------------ life of a request

    def add_request(self, rid: Hashable) -> RequestCache:
        if rid in self._requests:
            raise CacheError("request %r already holds cache" % (rid,))
        if not self._free_slots:
            raise OutOfPages("all %d state slots are taken" % self.num_state_slots)
        rc = RequestCache(rid, self._free_slots.pop(), tables=[[] for _ in self.groups],
                          first_live=[0 for _ in self.groups])
        self._requests[rid] = rc
        return rc

    def append(self, rid: Hashable, n_new: int) -> int:
        """Make room for the next ``n_new`` tokens of ``rid`` in every group; returns the position of
        the first of them. All or nothing: on OutOfPages nothing is taken."""
        if n_new <= 0:
            raise ValueError("append needs n_new > 0")
        rc = self.request(rid)
        if rc.pending:
            raise CacheError("request %r has an uncommitted append" % (rid,))
        need = self.pages_needed(rid, n_new)
        for gi, n in enumerate(need):
            if n > self.pools[gi].num_free:
                raise OutOfPages("request %r needs %d pages of group %d, %d are free"
                                 % (rid, n, gi, self.pools[gi].num_free))
        for gi, n in enumerate(need):
            for _ in range(n):
                rc.tables[gi].append(self.pools[gi].allocate())
        rc.pending = n_new
        return rc.num_tokens

    def commit(self, rid: Hashable) -> None:
        """The appended tokens are in the pages now. Pages a window has passed are given back."""
        rc = self.request(rid)
        rc.num_tokens += rc.pending
        rc.pending = 0
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            # the next query stands at position >= num_tokens and reads keys > num_tokens - window
            first_needed = max(0, rc.num_tokens - g.window + 1)
            keep_from = first_needed // g.page_size
            table = rc.tables[gi]
            for b in range(rc.first_live[gi], min(keep_from, len(table))):
                if table[b] != RELEASED:
                    self.pools[gi].release(table[b])
                    table[b] = RELEASED
            rc.first_live[gi] = max(rc.first_live[gi], min(keep_from, len(table)))

    def rollback(self, rid: Hashable) -> None:
        """Undo an append that was not committed: its pages go back."""
        rc = self.request(rid)
        if not rc.pending:
            return
        rc.pending = 0
        for gi, g in enumerate(self.groups):
            keep = -(-rc.num_tokens // g.page_size)
            table = rc.tables[gi]
            while len(table) > keep:
                p = table.pop()
                if p != RELEASED:
                    self.pools[gi].release(p)

    def free_request(self, rid: Hashable) -> None:
        """Give back everything ``rid`` holds."""
        rc = self.request(rid)
        for gi, table in enumerate(rc.tables):
            for p in reversed(table):
                if p != RELEASED:
                    self.pools[gi].release(p)
        self._free_slots.append(rc.state_slot)
        del self._requests[rid]

    def reset(self) -> None:
        for rid in list(self._requests):
            self.free_request(rid)

    # ------------------------------------------------------------------ what a step needs

    def slot_mapping(self, rid: Hashable, group: int, start: int, n: int) -> List[int]:
        """Slot (page * page_size + offset) of positions start .. start + n - 1 in ``group``."""
        rc = self.request(rid)
        ps = self.groups[group].page_size
        table = rc.tables[group]
        out = []
        for pos in range(start, start + n):
            page = table[pos // ps]
            if page == RELEASED:
                raise CacheError("position %d of request %r lies in a page that was given back" % (pos, rid))
            out.append(page * ps + pos % ps)
        return out

    def block_table(self, rid: Hashable, group: int) -> List[int]:
        """Page of every logical block of ``rid`` (RELEASED where the window has passed)."""
        return list(self.request(rid).tables[group])

    # ------------------------------------------------------------------ invariants (tests)

    def check_invariants(self) -> None:
        """No page lost or held twice; every live request's state slot is its own."""
        for gi, pool in enumerate(self.pools):
            held_by_tables = []
            for rc in self._requests.values():
                held_by_tables.extend(p for p in rc.tables[gi] if p != RELEASED)
            if len(held_by_tables) != len(set(held_by_tables)):
                raise CacheError("group %d: a page is in two block tables" % gi)
            for p in held_by_tables:
                if not pool.is_held(p):
                    raise CacheError("group %d: page %d is in a table but marked free" % (gi, p))
            if len(held_by_tables) + pool.num_free != pool.num_pages:
                raise CacheError("group %d: %d pages in tables + %d free != %d" %
                                 (gi, len(held_by_tables), pool.num_free, pool.num_pages))
            if len(set(pool._free)) != len(pool._free):
                raise CacheError("group %d: a page is on the free list twice" % gi)
        slots = [rc.state_slot for rc in self._requests.values()]
        if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots):
            raise CacheError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.num_state_slots:
            raise CacheError("state slots lost")
