"""Host side of the cache: page pools, block tables and state slots. No tensors here.

The work is done by the C++ cache manager of the host library (``lmsf_amd/csrc/host/cache_manager.cc``,
where the design and its relation to the reference's block manager are written down); this module is its
Python face: request ids of any hashable kind are mapped to the integers the library knows, its status
codes become ``OutOfPages`` / ``CacheError`` / ``ValueError``.

- Layers with equal needs form a *group* with a page pool and per-request block tables of its own; a
  group is either "full" (every key stays) or has a window W (only positions > p - W are read by a
  query at p).
- Pages are given back when a request ends, and, in a window group, as soon as the window has passed
  them. A freed page is the next one handed out (LIFO), so reuse is immediate.
- Beside the pages there are slots for per-request state of fixed size: one slot per live request,
  taken at its first tokens and given back with its pages.
- Nothing is shared between requests, so a page has one holder or none; giving back a page that is not
  held is an error.
"""
import ctypes
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np

from ..host import library as _host


class OutOfPages(RuntimeError):
    """A pool cannot supply the pages (or state slots) that an append needs."""


class CacheError(RuntimeError):
    """Misuse of the cache manager: unknown request, double free, a page held twice."""


def _raise(lib, status: int, who: str = "") -> None:
    msg = _host.last_error(lib)
    if who:
        msg = "%s: %s" % (who, msg)
    if status == _host.OUT_OF_PAGES:
        raise OutOfPages(msg)
    if status == _host.CACHE_ERROR:
        raise CacheError(msg)
    raise ValueError(msg)


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


class PagePool:
    """``num_pages`` page ids with a LIFO free list and a holder check."""

    def __init__(self, num_pages: int):
        self._lib = _host.load_host_library()
        self.num_pages = int(num_pages)
        h = ctypes.c_void_p()
        rc = self._lib.lmsf_pool_create(self.num_pages, ctypes.byref(h))
        if rc:
            _raise(self._lib, rc)
        self._h = h

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.lmsf_pool_destroy(self._h)
            self._h = None

    @property
    def num_free(self) -> int:
        return self._lib.lmsf_pool_num_free(self._h)

    def allocate(self) -> int:
        page = ctypes.c_int()
        rc = self._lib.lmsf_pool_allocate(self._h, ctypes.byref(page))
        if rc:
            _raise(self._lib, rc)
        return page.value

    def release(self, page: int) -> None:
        rc = self._lib.lmsf_pool_release(self._h, int(page))
        if rc:
            _raise(self._lib, rc)


@dataclass(frozen=True)
class GroupConfig:
    """One cache group: its page geometry and whether it keeps all keys or a window of them."""

    page_size: int
    num_pages: int
    window: Optional[int] = None


RELEASED = -1


@dataclass
class RequestCache:
    """What one live request holds (a copy, taken when it was asked for)."""

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
        self._lib = _host.load_host_library()
        self.groups = list(groups)
        self.num_state_slots = int(num_state_slots)
        G = len(self.groups)
        ps = np.asarray([g.page_size for g in self.groups], dtype=np.int32)
        npg = np.asarray([g.num_pages for g in self.groups], dtype=np.int32)
        win = np.asarray([g.window or 0 for g in self.groups], dtype=np.int32)
        h = ctypes.c_void_p()
        rc = self._lib.lmsf_cm_create(G, _ptr(ps), _ptr(npg), _ptr(win), self.num_state_slots, ctypes.byref(h))
        if rc:
            _raise(self._lib, rc)
        self._h = h
        # request ids of any hashable kind <-> the integers of the library
        self._handle_of: Dict[Hashable, int] = {}
        self._rid_of: Dict[int, Hashable] = {}
        self._pinned: Dict[Hashable, int] = {}      # ids another owner (the scheduler) wants kept
        self._next_handle = 1
        self._need = np.zeros(max(G, 1), dtype=np.int32)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.lmsf_cm_destroy(self._h)
            self._h = None

    # ------------------------------------------------------------------ ids

    @property
    def native(self) -> ctypes.c_void_p:
        """The library's object, for the other parts of the host library (scheduler, step metadata)."""
        return self._h

    def handle(self, rid: Hashable) -> int:
        """The library's integer for ``rid`` (a new one if it has none yet)."""
        h = self._handle_of.get(rid)
        if h is None:
            h = self._next_handle
            self._next_handle += 1
            self._handle_of[rid] = h
            self._rid_of[h] = rid
        return h

    def request_id(self, handle: int) -> Hashable:
        return self._rid_of[handle]

    def known_handle(self, rid: Hashable) -> Optional[int]:
        """The library's integer for ``rid`` if it has one."""
        return self._handle_of.get(rid)

    def pin(self, rid: Hashable) -> int:
        """Keep ``rid``'s integer also while it holds no cache (a request that waits); returns it."""
        self._pinned[rid] = self._pinned.get(rid, 0) + 1
        return self.handle(rid)

    def unpin(self, rid: Hashable) -> None:
        n = self._pinned.get(rid, 0) - 1
        if n > 0:
            self._pinned[rid] = n
            return
        self._pinned.pop(rid, None)
        self._forget_if_unused(rid)

    def _forget_if_unused(self, rid: Hashable) -> None:
        h = self._handle_of.get(rid)
        if h is not None and rid not in self._pinned and not self._lib.lmsf_cm_has_request(self._h, h):
            del self._handle_of[rid]
            del self._rid_of[h]

    def forget_released(self) -> None:
        """Drop the integers of requests that the library released on its own (the scheduler frees what a
        preempted or finished request holds)."""
        for rid in [r for r in self._handle_of if r not in self._pinned]:
            self._forget_if_unused(rid)

    def _known(self, rid: Hashable) -> Optional[int]:
        h = self._handle_of.get(rid)
        if h is not None and self._lib.lmsf_cm_has_request(self._h, h):
            return h
        return None

    def _must(self, rid: Hashable) -> int:
        h = self._known(rid)
        if h is None:
            raise CacheError("request %r holds no cache" % (rid,))
        return h

    # ------------------------------------------------------------------ queries

    def has_request(self, rid: Hashable) -> bool:
        return self._known(rid) is not None

    def request(self, rid: Hashable) -> RequestCache:
        h = self._must(rid)
        info = np.zeros(3, dtype=np.int64)
        rc = self._lib.lmsf_cm_request_info(self._h, h, _ptr(info))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))
        tables, first_live = [], []
        for gi in range(len(self.groups)):
            t, fl = self._table(h, gi)
            tables.append(t)
            first_live.append(fl)
        return RequestCache(rid, int(info[0]), int(info[1]), int(info[2]), tables, first_live)

    def state_slot(self, rid: Hashable) -> int:
        """The state slot that the live request ``rid`` holds."""
        info = np.zeros(3, dtype=np.int64)
        rc = self._lib.lmsf_cm_request_info(self._h, self._must(rid), _ptr(info))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))
        return int(info[0])

    def _table(self, h: int, group: int):
        n, fl = ctypes.c_int(), ctypes.c_int()
        rc = self._lib.lmsf_cm_block_table(self._h, h, group, None, 0, ctypes.byref(n), ctypes.byref(fl))
        if rc:
            _raise(self._lib, rc)
        out = np.zeros(max(n.value, 1), dtype=np.int32)
        rc = self._lib.lmsf_cm_block_table(self._h, h, group, _ptr(out), out.shape[0], ctypes.byref(n), ctypes.byref(fl))
        if rc:
            _raise(self._lib, rc)
        return out[:n.value].tolist(), fl.value

    def live_requests(self) -> List[Hashable]:
        n = ctypes.c_int()
        self._lib.lmsf_cm_live_requests(self._h, None, 0, ctypes.byref(n))
        out = np.zeros(max(n.value, 1), dtype=np.int64)
        self._lib.lmsf_cm_live_requests(self._h, _ptr(out), out.shape[0], ctypes.byref(n))
        return [self._rid_of[int(h)] for h in out[:n.value]]

    def num_free_pages(self, group: int = 0) -> int:
        n = ctypes.c_int()
        rc = self._lib.lmsf_cm_num_free_pages(self._h, int(group), ctypes.byref(n))
        if rc:
            _raise(self._lib, rc)
        return n.value

    def num_free_state_slots(self) -> int:
        return self._lib.lmsf_cm_num_free_state_slots(self._h)

    def num_tokens(self, rid: Hashable) -> int:
        info = np.zeros(3, dtype=np.int64)
        rc = self._lib.lmsf_cm_request_info(self._h, self._must(rid), _ptr(info))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))
        return int(info[1])

    def tokens_held(self, rids: Sequence[Hashable]) -> np.ndarray:
        """``num_tokens`` of every request of the list at once (0 for one that holds no cache)."""
        S = len(rids)
        get = self._handle_of.get
        handles = np.fromiter((get(r, -1) for r in rids), dtype=np.int64, count=S)
        known = (handles >= 0).astype(np.uint8)
        held = np.zeros(max(S, 1), dtype=np.int64)
        rc = self._lib.lmsf_cm_tokens_held(self._h, S, _ptr(handles), _ptr(known), _ptr(held))
        if rc:
            _raise(self._lib, rc)
        return held[:S]

    def pages_needed(self, rid: Optional[Hashable], n_new: int, held_tokens: Optional[int] = None) -> List[int]:
        """New pages per group that appending ``n_new`` tokens would take. ``rid`` None (or unknown)
        counts for a request that holds nothing yet."""
        h = self._known(rid) if rid is not None else None
        rc = self._lib.lmsf_cm_pages_needed(self._h, 0 if h is None else 1, h or 0, int(n_new), _ptr(self._need))
        if rc:
            _raise(self._lib, rc)
        return self._need[:len(self.groups)].tolist()

    def can_append(self, rid: Optional[Hashable], n_new: int, reserve_pages: int = 0) -> bool:
        """True if ``n_new`` more tokens of ``rid`` fit, leaving ``reserve_pages`` free in every group."""
        h = self._known(rid) if rid is not None else None
        return self._lib.lmsf_cm_can_append(self._h, 0 if h is None else 1, h or 0, int(n_new), int(reserve_pages)) == 1

    # ------------------------------------------------------------------ life of a request

    def add_request(self, rid: Hashable) -> RequestCache:
        if self._known(rid) is not None:
            raise CacheError("request %r already holds cache" % (rid,))
        slot = ctypes.c_int()
        rc = self._lib.lmsf_cm_add_request(self._h, self.handle(rid), ctypes.byref(slot))
        if rc:
            self._forget_if_unused(rid)
            _raise(self._lib, rc, "request %r" % (rid,))
        G = len(self.groups)
        return RequestCache(rid, slot.value, tables=[[] for _ in range(G)], first_live=[0] * G)

    def append(self, rid: Hashable, n_new: int) -> int:
        """Make room for the next ``n_new`` tokens of ``rid`` in every group; returns the position of
        the first of them. All or nothing: on OutOfPages nothing is taken."""
        if n_new <= 0:
            raise ValueError("append needs n_new > 0")
        start = ctypes.c_int64()
        rc = self._lib.lmsf_cm_append(self._h, self._must(rid), int(n_new), ctypes.byref(start))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))
        return start.value

    def commit(self, rid: Hashable) -> None:
        """The appended tokens are in the pages now. Pages a window has passed are given back."""
        rc = self._lib.lmsf_cm_commit(self._h, self._must(rid))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))

    def rollback(self, rid: Hashable) -> None:
        """Undo an append that was not committed: its pages go back."""
        rc = self._lib.lmsf_cm_rollback(self._h, self._must(rid))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))

    def free_request(self, rid: Hashable) -> None:
        """Give back everything ``rid`` holds."""
        rc = self._lib.lmsf_cm_free_request(self._h, self._must(rid))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))
        self._forget_if_unused(rid)

    def reset(self) -> None:
        rc = self._lib.lmsf_cm_reset(self._h)
        if rc:
            _raise(self._lib, rc)
        self.forget_released()

    # ------------------------------------------------------------------ what a step needs

    def slot_mapping(self, rid: Hashable, group: int, start: int, n: int) -> List[int]:
        """Slot (page * page_size + offset) of positions start .. start + n - 1 in ``group``."""
        out = np.zeros(max(int(n), 1), dtype=np.int32)
        rc = self._lib.lmsf_cm_slot_mapping(self._h, self._must(rid), int(group), int(start), int(n), _ptr(out))
        if rc:
            _raise(self._lib, rc, "request %r" % (rid,))
        return out[:n].tolist()

    def block_table(self, rid: Hashable, group: int) -> List[int]:
        """Page of every logical block of ``rid`` (RELEASED where the window has passed)."""
        return self._table(self._must(rid), int(group))[0]

    def begin_step(self, rids: Sequence[Hashable], lens: Sequence[int]):
        """Add the requests that hold nothing yet and append every entry's tokens, all or nothing (on
        OutOfPages nothing is taken). Returns (handles, first positions, which were added) as arrays for
        ``abort_step`` / ``commit_step`` / ``fill_step``."""
        S = len(rids)
        handles = np.fromiter((self.handle(r) for r in rids), dtype=np.int64, count=S)
        lens_a = np.asarray(lens, dtype=np.int32)
        starts = np.zeros(S, dtype=np.int64)
        added = np.zeros(S, dtype=np.uint8)
        rc = self._lib.lmsf_cm_begin_step(self._h, S, _ptr(handles), _ptr(lens_a), _ptr(starts), _ptr(added))
        if rc:
            for r in rids:
                self._forget_if_unused(r)
            _raise(self._lib, rc)
        return handles, starts, added

    def abort_step(self, rids: Sequence[Hashable], handles: np.ndarray, added: np.ndarray) -> None:
        """The step failed after ``begin_step``: what it took goes back."""
        rc = self._lib.lmsf_cm_abort_step(self._h, len(rids), _ptr(handles), _ptr(added))
        for r in rids:
            self._forget_if_unused(r)
        if rc:
            _raise(self._lib, rc)

    def commit_step(self, handles: np.ndarray) -> None:
        rc = self._lib.lmsf_cm_commit_step(self._h, int(handles.shape[0]), _ptr(handles))
        if rc:
            _raise(self._lib, rc)

    def step_widths(self, handles: np.ndarray) -> List[int]:
        """Per group, the longest block table among these requests (at least 1)."""
        w = np.zeros(max(len(self.groups), 1), dtype=np.int32)
        rc = self._lib.lmsf_cm_step_widths(self._h, int(handles.shape[0]), _ptr(handles), _ptr(w))
        if rc:
            _raise(self._lib, rc)
        return w[:len(self.groups)].tolist()

    def step_layout(self, N: int, S: int, R: int, widths: Sequence[int]):
        """Offsets (int32 elements, 16-byte aligned) of the sections of a step's metadata buffer, by name,
        as (offset, length); the raw offsets for ``fill_step``; and the buffer's size."""
        G = len(widths)
        w = np.asarray(list(widths) or [0], dtype=np.int32)
        raw = np.zeros(7 + 2 * G, dtype=np.int64)
        total = ctypes.c_int64()
        rc = self._lib.lmsf_step_layout(int(N), int(S), int(R), G, _ptr(w), _ptr(raw), ctypes.byref(total))
        if rc:
            _raise(self._lib, rc)
        names = [("token_ids", N), ("positions", N), ("seg_of", N), ("seg_starts", S + 1), ("seg_first", S),
                 ("state_slots", S), ("logit_rows", R)]
        for gi in range(G):
            names += [("slots%d" % gi, N), ("tables%d" % gi, S * int(widths[gi]))]
        offsets = {name: (int(raw[i]), int(n)) for i, (name, n) in enumerate(names)}
        return offsets, raw, int(total.value)

    def fill_step(self, handles: np.ndarray, starts: np.ndarray, lens: Sequence[int], widths: Sequence[int],
                  raw_offsets: np.ndarray, buffer: np.ndarray) -> None:
        """Write positions, segments, state slots, slots and block tables of a step into its metadata
        buffer (int32); token ids and logit rows are the caller's. Pages that a window has passed appear as
        page 0 in the tables; a token whose own page was given back is an error."""
        lens_a = np.asarray(lens, dtype=np.int32)
        w = np.asarray(list(widths) or [0], dtype=np.int32)
        if buffer.dtype != np.int32 or not buffer.flags["C_CONTIGUOUS"]:
            raise ValueError("the metadata buffer must be contiguous int32")
        rc = self._lib.lmsf_cm_fill_step(self._h, int(handles.shape[0]), _ptr(handles), _ptr(starts), _ptr(lens_a),
                                         _ptr(w), _ptr(raw_offsets), _ptr(buffer))
        if rc:
            _raise(self._lib, rc)

    # ------------------------------------------------------------------ invariants (tests)

    def check_invariants(self) -> None:
        """No page lost or held twice; every live request's state slot is its own."""
        rc = self._lib.lmsf_cm_check_invariants(self._h)
        if rc:
            _raise(self._lib, rc)
