"""The scheduler in plain Python: the oracle that the C++ scheduler of the host library is checked
against, plan by plan, over random workloads.

Continuous batching above the step function: admits requests, cuts prompts into portions under
a token budget, decodes, and decides what happens when pages run out.

The reference's scheduler (core/src/sched/scheduler.rs:343-543) runs either a batch of whole
prompts or a batch of decode tokens, admits a prompt only when all its blocks fit
(core/src/sched/block_manager.rs:104-122), and on shortage preempts the latest arrival by
recompute (:253-284, :459-490). Kept from it: first come first served by arrival, head-of-line
admission with a watermark of free pages, preemption by recompute of the latest arrival with
re-insertion at the front of the waiting queue, and prompts longer than the limit being ignored
(:368-381). Different: a step holds real tokens under ``max_num_batched_tokens``: first one token
for every decoding request, then portions of prompts in arrival order, each at most
``prefill_chunk_size`` long.

What happens when pages run out is written out once, at the top of lmsf_amd/csrc/host/scheduler.h.
"""
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Hashable, List, Optional

from plain_cache_manager import CacheManager
from lmsf_amd.engine.sequence import Sequence, SequenceState


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
        self.waiting: Deque[Sequence] = deque()
        self.running: List[Sequence] = []
        self.num_preemptions = 0

    # ------------------------------------------------------------------ queue operations

    def add(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def abort(self, request_id: Hashable) -> Optional[Sequence]:
        """core/src/sched/scheduler.rs:160-196: by request id, in whichever queue."""
        for q in (self.waiting, self.running):
            for seq in list(q):
                if seq.request_id == request_id:
                    q.remove(seq)
                    seq.state = SequenceState.FINISHED_ABORTED
                    self._release(seq)
                    return seq
        return None

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def num_unfinished(self) -> int:
        return len(self.waiting) + len(self.running)

    def finish(self, seq: Sequence) -> None:
        """The engine decided that ``seq`` is done: drop it and give back what it holds."""
        if seq in self.running:
            self.running.remove(seq)
        if seq in self.waiting:           # preempted after its last token had been sampled
            self.waiting.remove(seq)
        self._release(seq)

    def _release(self, seq: Sequence) -> None:
        if self.cache.has_request(seq.request_id):
            self.cache.free_request(seq.request_id)

    # ------------------------------------------------------------------ planning

    def schedule(self) -> StepPlan:
        cfg, cache = self.config, self.cache
        plan = StepPlan()
        budget = cfg.max_num_batched_tokens
        planned = [0] * len(cache.groups)          # pages promised to earlier entries of this plan
        planned_slots = 0
        watermark = [int(round(cfg.watermark * g.num_pages)) for g in cache.groups]

        last_need = [None, None, None]             # (request, tokens) of the last question and its answer

        def needed(rid, n):
            if last_need[0] != rid or last_need[1] != n or rid is None:
                last_need[0], last_need[1], last_need[2] = rid, n, cache.pages_needed(rid, n)
            return last_need[2]

        def fits(rid, n, reserve=False) -> bool:
            for gi, k in enumerate(needed(rid, n)):
                if cache.num_free_pages(gi) - planned[gi] - k < (watermark[gi] if reserve else 0):
                    return False
            return True

        def take(rid, n) -> None:
            for gi, k in enumerate(needed(rid, n)):
                planned[gi] += k

        self.running.sort(key=lambda s: s.arrival)
        # two passes over the running requests, each in arrival order: the decoding requests get their token
        # first (core/src/sched/scheduler.rs:459-490), prompts are cut from the budget that is left
        unserved = list(self.running)

        def run_one(seq) -> None:
            nonlocal budget
            unserved.remove(seq)
            decoding = seq.remaining == 1
            n = 1 if decoding else min(seq.remaining, budget, cfg.prefill_chunk_size or seq.remaining)
            while not fits(seq.request_id, n):
                if n > 1:
                    room = min(self._room_tokens(seq, planned), n - 1)      # a shorter portion may fit
                    if room >= 1:
                        n = room
                        continue
                behind = [s for s in unserved if s.arrival > seq.arrival]
                if behind:
                    victim = max(behind, key=lambda s: s.arrival)           # the latest arrival
                    unserved.remove(victim)
                    self._preempt(victim, plan)
                    continue
                if not plan.scheduled and not unserved:
                    # alone and still no room: it can never continue
                    self.running.remove(seq)
                    seq.state = SequenceState.FINISHED_LENGTH_CAPPED
                    self._release(seq)
                    plan.capped.append(seq)
                elif decoding:
                    self._preempt(seq, plan)
                # else: a prompt with nobody behind it waits, keeping its pages
                return
            take(seq.request_id, n)
            plan.scheduled.append(ScheduledSequence(seq, seq.num_computed, n, seq.num_computed + n == seq.length))
            budget -= n

        for want_decoding in (True, False):
            for seq in list(self.running):
                if budget <= 0:
                    break
                if seq in unserved and (seq.remaining == 1 or not want_decoding):
                    run_one(seq)

        # admission, head of line only; nothing is admitted in a step that had to preempt
        while self.waiting and not plan.preempted and budget > 0 and \
                len(self.running) < cfg.max_num_seqs:
            seq = self.waiting[0]
            limit = min(cfg.max_model_len, cache_capacity_tokens(cache))
            if seq.length > limit or seq.length == 0:
                self.waiting.popleft()
                seq.state = SequenceState.FINISHED_IGNORED
                plan.ignored.append(seq)
                continue
            if cache.num_free_state_slots() - planned_slots <= 0:
                break
            n = min(seq.remaining, budget, cfg.prefill_chunk_size or seq.remaining)
            if not fits(None, n, reserve=True):
                room = min(self._room_tokens(None, planned, watermark), n)
                idle = not self.running and not plan.scheduled
                if room < 1:
                    if not idle:
                        break                      # wait for pages
                    # every page is free and not one token fits above the watermark: it never will
                    self.waiting.popleft()
                    seq.state = SequenceState.FINISHED_IGNORED
                    plan.ignored.append(seq)
                    continue
                if room < min(n, 16) and not idle:
                    break                          # wait for pages rather than crawl
                n = room
            self.waiting.popleft()
            take(None, n)
            planned_slots += 1
            seq.state = SequenceState.RUNNING
            if seq.metrics.first_scheduled_time is None:
                seq.metrics.first_scheduled_time = time.monotonic()
            self.running.append(seq)
            plan.scheduled.append(ScheduledSequence(seq, seq.num_computed, n, seq.num_computed + n == seq.length))
            budget -= n
        return plan

    def _room_tokens(self, seq: Optional[Sequence], planned: List[int], watermark: Optional[List[int]] = None) -> int:
        """How many more tokens of ``seq`` (None: a new request) fit in the pages that are free now."""
        cache = self.cache
        room = None
        for gi, g in enumerate(cache.groups):
            free = cache.num_free_pages(gi) - planned[gi] - (watermark[gi] if watermark else 0)
            held = 0
            slack = 0
            if seq is not None and cache.has_request(seq.request_id):
                rc = cache.request(seq.request_id)
                held = rc.num_tokens
                slack = len(rc.tables[gi]) * g.page_size - held
            r = max(0, free) * g.page_size + slack
            room = r if room is None else min(room, r)
        return room or 0

    def _preempt(self, seq: Sequence, plan: StepPlan) -> None:
        """Preemption by recompute (core/src/sched/scheduler.rs:274-284): everything the request holds
        goes back, and it returns to the front of the waiting queue."""
        if seq in self.running:
            self.running.remove(seq)
        if seq in self.waiting:           # preempted after its last token had been sampled
            self.waiting.remove(seq)
        self._release(seq)
        seq.num_computed = 0
        seq.num_preemptions += 1
        seq.state = SequenceState.WAITING
        self.waiting.appendleft(seq)
        plan.preempted.append(seq)
        self.num_preemptions += 1


def cache_capacity_tokens(cache: CacheManager) -> int:
    """Tokens one request could hold if it had every page of the groups that keep all keys."""
    caps = [g.num_pages * g.page_size for g in cache.groups if g.window is None]
    return min(caps) if caps else 1 << 62
