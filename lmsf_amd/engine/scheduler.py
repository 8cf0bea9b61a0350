"""Continuous batching above the step function: admits requests, cuts prompts into portions under
a token budget, decodes, and decides what happens when pages run out.

The decisions are made by the C++ scheduler of the host library (``lmsf_amd/csrc/host/scheduler.cc``;
its header says what is kept from the reference's scheduler, core/src/sched/scheduler.rs:343-543, and
what is different). This module is its Python face: it owns the ``Sequence`` objects (token ids,
sampling parameters), tells the library each request's length and progress before a plan is made, and
writes the plan's consequences (state, progress, counters) back to them.

What happens when pages run out is written out once, at the top of ``lmsf_amd/csrc/host/scheduler.h``.
"""
import ctypes
import time
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional

import numpy as np

from ..cache.manager import CacheManager, _ptr, _raise
from ..host import library as _host
from .sequence import Sequence, SequenceState


@dataclass
class SchedulerConfig:
    """core/src/common/config.rs:287-314."""
    max_num_batched_tokens: int
    max_num_seqs: int
    max_model_len: int
    prefill_chunk_size: Optional[int] = None      # None: a portion is as long as the budget allows
    watermark: float = 0.01                       # share of pages kept free at admission (block_manager.rs:88)

    def __post_init__(self):
        if self.max_num_batched_tokens <= 0 or self.max_num_seqs <= 0 or self.max_model_len <= 0:
            raise ValueError("scheduler limits must be > 0")
        if self.prefill_chunk_size is not None and self.prefill_chunk_size <= 0:
            raise ValueError("prefill_chunk_size must be > 0")


@dataclass
class ScheduledSequence:
    seq: Sequence
    start: int          # position of the first token of this portion
    n_tokens: int
    samples: bool       # the portion ends at the request's last token: a token is sampled after it


@dataclass
class StepPlan:
    scheduled: List[ScheduledSequence] = field(default_factory=list)
    preempted: List[Sequence] = field(default_factory=list)
    ignored: List[Sequence] = field(default_factory=list)       # finished without running (too long)
    capped: List[Sequence] = field(default_factory=list)        # finished for lack of pages while alone

    @property
    def num_tokens(self) -> int:
        return sum(s.n_tokens for s in self.scheduled)

    @property
    def empty(self) -> bool:
        return not self.scheduled


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache: CacheManager):
        self.config = config
        self.cache = cache
        self._lib = _host.load_host_library()
        h = ctypes.c_void_p()
        rc = self._lib.lmsf_sched_create(cache.native, int(config.max_num_batched_tokens), int(config.max_num_seqs),
                                         int(config.max_model_len), int(config.prefill_chunk_size or 0),
                                         float(config.watermark), ctypes.byref(h))
        if rc:
            _raise(self._lib, rc)
        self._h = h
        self._seqs: Dict[int, Sequence] = {}        # the library's integer -> the request, while it is scheduled

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.lmsf_sched_destroy(self._h)
            self._h = None

    # ------------------------------------------------------------------ queue operations

    def add(self, seq: Sequence) -> None:
        h = self.cache.pin(seq.request_id)
        rc = self._lib.lmsf_sched_add(self._h, h, int(seq.arrival), int(seq.length))
        if rc:
            self.cache.unpin(seq.request_id)
            _raise(self._lib, rc, "request %r" % (seq.request_id,))
        self._seqs[h] = seq

    def _drop(self, h: int) -> Optional[Sequence]:
        seq = self._seqs.pop(h, None)
        if seq is not None:
            self.cache.unpin(seq.request_id)
        return seq

    def _handle(self, request_id: Hashable) -> Optional[int]:
        h = self.cache.known_handle(request_id)
        return h if h in self._seqs else None

    def abort(self, request_id: Hashable) -> Optional[Sequence]:
        """core/src/sched/scheduler.rs:160-196: by request id, in whichever queue."""
        h = self._handle(request_id)
        if h is None:
            return None
        found = ctypes.c_int()
        rc = self._lib.lmsf_sched_abort(self._h, h, ctypes.byref(found))
        if rc:
            _raise(self._lib, rc)
        seq = self._drop(h)
        seq.state = SequenceState.FINISHED_ABORTED
        return seq

    def has_unfinished(self) -> bool:
        return bool(self._seqs)

    def num_unfinished(self) -> int:
        return len(self._seqs)

    def finish(self, seq: Sequence) -> None:
        """The engine decided that ``seq`` is done: drop it and give back what it holds."""
        h = self._handle(seq.request_id)
        if h is None:
            return
        rc = self._lib.lmsf_sched_finish(self._h, h)
        if rc:
            _raise(self._lib, rc)
        self._drop(h)

    def _queue(self, which: int) -> List[Sequence]:
        n = ctypes.c_int()
        self._lib.lmsf_sched_queue(self._h, which, None, 0, ctypes.byref(n))
        out = np.zeros(max(n.value, 1), dtype=np.int64)
        self._lib.lmsf_sched_queue(self._h, which, _ptr(out), out.shape[0], ctypes.byref(n))
        return [self._seqs[int(h)] for h in out[:n.value]]

    @property
    def waiting(self) -> List[Sequence]:
        """The waiting requests, the head of the line first."""
        return self._queue(0)

    @property
    def running(self) -> List[Sequence]:
        return self._queue(1)

    @property
    def num_preemptions(self) -> int:
        return int(self._lib.lmsf_sched_num_preemptions(self._h))

    # ------------------------------------------------------------------ planning

    def schedule(self) -> StepPlan:
        n = len(self._seqs)
        if n:
            ids = np.fromiter(self._seqs.keys(), dtype=np.int64, count=n)
            lengths = np.fromiter((s.length for s in self._seqs.values()), dtype=np.int64, count=n)
            computed = np.fromiter((s.num_computed for s in self._seqs.values()), dtype=np.int64, count=n)
            rc = self._lib.lmsf_sched_set_progress(self._h, n, _ptr(ids), _ptr(lengths), _ptr(computed))
            if rc:
                _raise(self._lib, rc)
        counts = np.zeros(4, dtype=np.int32)
        rc = self._lib.lmsf_sched_schedule(self._h, _ptr(counts))
        if rc:
            _raise(self._lib, rc)
        ns, npre, nig, ncap = (int(c) for c in counts)
        ids, starts, toks = (np.zeros(max(ns, 1), dtype=np.int64) for _ in range(3))
        samples = np.zeros(max(ns, 1), dtype=np.int32)
        pre, ign, cap = (np.zeros(max(k, 1), dtype=np.int64) for k in (npre, nig, ncap))
        rc = self._lib.lmsf_sched_plan(self._h, _ptr(ids), _ptr(starts), _ptr(toks), _ptr(samples), _ptr(pre), _ptr(ign),
                                       _ptr(cap))
        if rc:
            _raise(self._lib, rc)
        plan = StepPlan()
        for h in pre[:npre]:
            seq = self._seqs[int(h)]
            seq.num_computed = 0
            seq.num_preemptions += 1
            seq.state = SequenceState.WAITING
            plan.preempted.append(seq)
        for h in ign[:nig]:
            seq = self._drop(int(h))
            seq.state = SequenceState.FINISHED_IGNORED
            plan.ignored.append(seq)
        for h in cap[:ncap]:
            seq = self._drop(int(h))
            seq.state = SequenceState.FINISHED_LENGTH_CAPPED
            plan.capped.append(seq)
        for i in range(ns):
            seq = self._seqs[int(ids[i])]
            if seq.state != SequenceState.RUNNING:
                seq.state = SequenceState.RUNNING
                if seq.metrics.first_scheduled_time is None:
                    seq.metrics.first_scheduled_time = time.monotonic()
            plan.scheduled.append(ScheduledSequence(seq, int(starts[i]), int(toks[i]), bool(samples[i])))
        if npre or ncap:
            self.cache.forget_released()
        return plan


def cache_capacity_tokens(cache: CacheManager) -> int:
    """Tokens one request could hold if it had every page of the groups that keep all keys."""
    caps = [g.num_pages * g.page_size for g in cache.groups if g.window is None]
    return min(caps) if caps else 1 << 62
