"""Device side of the cache: the page tensors of every cache group and the state slots.

The reference allocates per layer K [blocks, kv_heads, d/x, block, x] and V [blocks, kv_heads, d, block]
(core/src/worker/cache_engine.rs:107-160) and sizes the pool from free device memory
(core/src/worker/model_worker.rs:128-162, block bytes :cache_engine.rs:88-105). Here K is
[pages, kv_heads, page_size, head_dim] and V [pages, kv_heads, v_head_dim, page_size] (a value as wide as a key
unless the mixer says otherwise); runs of layers whose mixers declare equal needs form
a group that shares page ids, so one block table serves all of them.
"""
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import CacheBinding, CacheSpec, Runtime, StateSpec
from .manager import CacheManager, GroupConfig


@dataclass
class GroupLayout:
    spec: CacheSpec
    entries: List[int]            # schedule entries that own pages in this group
    page_size: int
    num_pages: int = 0

    def bytes_per_page(self, elem_size: int) -> int:
        return len(self.entries) * self.spec.num_kv_heads * self.page_size * (self.spec.head_dim + self.spec.value_dim) \
            * elem_size


def plan_groups(requirements: Sequence[Tuple[Optional[CacheSpec], Optional[StateSpec], Optional[int]]],
                page_size: int) -> Tuple[List[GroupLayout], List[Optional[int]]]:
    """Group the schedule entries by what their mixers need. Returns the groups and, per entry, the
    index of its group (None for a mixer without paged cache)."""
    groups: List[GroupLayout] = []
    by_spec: Dict[CacheSpec, int] = {}
    entry_group: List[Optional[int]] = []
    for i, (cspec, _, src) in enumerate(requirements):
        if cspec is None:
            entry_group.append(None)
            continue
        if src is not None:
            # reads another run's pages: same group as that run, whatever window it applies itself
            entry_group.append(entry_group[src])
            continue
        if cspec not in by_spec:
            by_spec[cspec] = len(groups)
            groups.append(GroupLayout(cspec, [], page_size))
        gi = by_spec[cspec]
        groups[gi].entries.append(i)
        entry_group.append(gi)
    return groups, entry_group


class CacheStorage:
    """Allocates pages and state for a model and binds every run of its schedule to them."""

    def __init__(self, model, rt: Runtime, page_size: int, num_pages: Sequence[int], num_state_slots: int):
        self.rt = rt
        self.page_size = int(page_size)
        reqs = model.cache_requirements()
        self.groups, self.entry_group = plan_groups(reqs, self.page_size)
        if len(num_pages) != len(self.groups):
            raise ValueError("%d cache groups, %d page counts given" % (len(self.groups), len(num_pages)))
        for g, n in zip(self.groups, num_pages):
            g.num_pages = int(n)
        self.num_state_slots = int(num_state_slots)
        self.spare_state_slot = self.num_state_slots
        self.manager = CacheManager([GroupConfig(g.page_size, g.num_pages, g.spec.window) for g in self.groups],
                                    self.num_state_slots)
        bindings: List[CacheBinding] = []
        for i, (cspec, sspec, src) in enumerate(reqs):
            b = CacheBinding()
            if cspec is not None:
                b.group = self.entry_group[i]
                if src is None:
                    g = self.groups[b.group]
                    n = max(1, g.num_pages)
                    b.k_pages = torch.zeros((n, cspec.num_kv_heads, g.page_size, cspec.head_dim), dtype=rt.dtype,
                                            device=rt.device)
                    b.v_pages = torch.zeros((n, cspec.num_kv_heads, cspec.value_dim, g.page_size), dtype=rt.dtype,
                                            device=rt.device)
                else:
                    b.k_pages, b.v_pages = bindings[src].k_pages, bindings[src].v_pages
                    b.writes_cache = False
            if sspec is not None:
                # one row more than there are slots: the spare one, for a padded batch's tokens that belong to
                # no request
                b.state = torch.zeros((self.num_state_slots + 1,) + tuple(sspec.shape), dtype=sspec.dtype,
                                      device=rt.device)
            bindings.append(b)
        self.bindings = bindings
        self.has_state = any(b.state is not None for b in bindings)
        model.bind_cache(bindings)

    def clear_state_slots(self, slots: Sequence[int]) -> None:
        """Zeroes these slots of every state tensor: a request that takes a slot finds no trace of the one that
        held it before (the reference has no per-request state; its block manager hands out blocks as they are,
        core/src/sched/block_manager.rs:29-43, which is right for keys that are written before they are read)."""
        states = {b.state.data_ptr(): b.state for b in self.bindings if b.state is not None}
        if not states or not len(slots):
            return
        idx = torch.as_tensor(list(slots), dtype=torch.long, device=self.rt.device)
        for st in states.values():
            st.index_fill_(0, idx, 0)

    def bytes_allocated(self) -> int:
        total = 0
        seen = set()
        for b in self.bindings:
            for t in (b.k_pages, b.v_pages, b.state):
                if t is not None and t.data_ptr() not in seen:
                    seen.add(t.data_ptr())
                    total += t.numel() * t.element_size()
        return total


def bytes_per_token(model, page_size: int, elem_size: int) -> int:
    """Cache bytes one token of context costs in the groups that keep every key."""
    groups, _ = plan_groups(model.cache_requirements(), page_size)
    return sum(g.bytes_per_page(elem_size) // page_size for g in groups if g.spec.window is None)
