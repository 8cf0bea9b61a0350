"""The C++ host library (cache manager, scheduler, step metadata) against the plain Python
implementations under ``tests/``: the same calls in random order must give the same answers."""
import random

import numpy as np
import pytest

import plain_cache_manager as plain_cm
import plain_scheduler as plain_sched
from lmsf_amd.cache import CacheError, CacheManager, GroupConfig, OutOfPages
from lmsf_amd.engine.scheduler import Scheduler, SchedulerConfig
from lmsf_amd.engine.sequence import Sequence
from lmsf_amd.sampling import SamplingParams


def both_managers(groups, slots):
    return (CacheManager([GroupConfig(*g) for g in groups], slots),
            plain_cm.CacheManager([plain_cm.GroupConfig(*g) for g in groups], slots))


def outcome(f, *args):
    """('ok', value) or the kind of error."""
    try:
        return ("ok", f(*args))
    except (OutOfPages, plain_cm.OutOfPages):
        return ("out_of_pages", None)
    except (CacheError, plain_cm.CacheError):
        return ("cache_error", None)
    except ValueError:
        return ("value_error", None)


def same_state(a, b, rids):
    assert sorted(a.live_requests(), key=str) == sorted(b.live_requests(), key=str)
    assert a.num_free_state_slots() == b.num_free_state_slots()
    for g in range(len(a.groups)):
        assert a.num_free_pages(g) == b.num_free_pages(g)
    for rid in rids:
        assert a.has_request(rid) == b.has_request(rid)
        if a.has_request(rid):
            ra, rb = a.request(rid), b.request(rid)
            assert (ra.state_slot, ra.num_tokens, ra.pending, ra.tables, ra.first_live) == \
                   (rb.state_slot, rb.num_tokens, rb.pending, rb.tables, rb.first_live)


@pytest.mark.parametrize("seed", range(10))
def test_cache_manager_equals_the_plain_one_under_random_calls(seed):
    rng = random.Random(seed)
    groups = [(rng.choice([1, 4, 16]), rng.randrange(4, 30), None),
              (rng.choice([2, 8]), rng.randrange(4, 30), rng.choice([3, 10, 33]))][:rng.choice([1, 2])]
    a, b = both_managers(groups, 4)
    rids = ["r%d" % i for i in range(6)] + [7, (1, 2)]
    for _ in range(800):
        rid = rng.choice(rids)
        op = rng.choice(["add", "append", "append", "commit", "commit", "rollback", "free", "needed", "can", "slots",
                         "table", "tokens"])
        if op == "add":
            ra, rb = outcome(a.add_request, rid), outcome(b.add_request, rid)
            assert ra[0] == rb[0]
            if ra[0] == "ok":
                assert ra[1].state_slot == rb[1].state_slot
        elif op == "append":
            n = rng.choice([0, 1, 1, 2, 5, 17, 40])
            assert outcome(a.append, rid, n) == outcome(b.append, rid, n)
        elif op in ("commit", "rollback", "free"):
            name = {"commit": "commit", "rollback": "rollback", "free": "free_request"}[op]
            assert outcome(getattr(a, name), rid) == outcome(getattr(b, name), rid)
        elif op == "needed":
            n = rng.randrange(0, 50)
            who = rng.choice([rid, None])
            assert a.pages_needed(who, n) == b.pages_needed(who, n)
        elif op == "can":
            n, reserve = rng.randrange(1, 50), rng.choice([0, 0, 1, 3])
            who = rng.choice([rid, None])
            assert a.can_append(who, n, reserve) == b.can_append(who, n, reserve)
        elif op == "slots" and b.has_request(rid):
            rc = b.request(rid)
            total = rc.num_tokens + rc.pending
            if total:
                start = rng.randrange(0, total)
                n = rng.randrange(1, total - start + 1)
                g = rng.randrange(len(groups))
                assert outcome(a.slot_mapping, rid, g, start, n) == outcome(b.slot_mapping, rid, g, start, n)
        elif op == "table":
            g = rng.randrange(len(groups))
            assert outcome(a.block_table, rid, g) == outcome(b.block_table, rid, g)
        elif op == "tokens":
            assert outcome(a.num_tokens, rid) == outcome(b.num_tokens, rid)
        a.check_invariants()
        b.check_invariants()
        same_state(a, b, rids)
    a.reset()
    b.reset()
    same_state(a, b, rids)
    assert not a._handle_of                    # no id is kept for a request that holds nothing


def make_seq(rid, n_prompt, arrival):
    return Sequence(rid, list(range(1, n_prompt + 1)), SamplingParams(max_tokens=1 << 30), arrival, seed=0)


def plan_as_data(plan):
    return ([(s.seq.request_id, s.start, s.n_tokens, s.samples) for s in plan.scheduled],
            [s.request_id for s in plan.preempted], [s.request_id for s in plan.ignored],
            [s.request_id for s in plan.capped])


def run_workload(seed):
    """Both schedulers see the same arrivals, finishes and aborts and must make the same plan in every step:
    the same portions in the same order, the same victims, the same refusals. Returns how often each kind
    of decision was met."""
    rng = random.Random(1000 + seed)
    ps = rng.choice([4, 16])
    groups = [(ps, rng.randrange(6, 40), None)]
    if rng.random() < 0.4:
        groups.append((rng.choice([2, 8]), rng.randrange(6, 30), rng.choice([5, 24])))
    slots = rng.choice([2, 4, 8])
    cfg = dict(max_num_batched_tokens=rng.choice([8, 32, 100]), max_num_seqs=slots, max_model_len=rng.choice([64, 300]),
               prefill_chunk_size=rng.choice([None, 7, 16]), watermark=rng.choice([0.01, 0.1]))
    ca, cb = both_managers(groups, slots)
    sa = Scheduler(SchedulerConfig(**cfg), ca)
    sb = plain_sched.Scheduler(plain_sched.SchedulerConfig(**cfg), cb)
    seqs_a, seqs_b = {}, {}
    arrivals = 0
    saw = {"preempted": 0, "ignored": 0, "capped": 0, "portions": 0}
    for step in range(250):
        for _ in range(rng.choice([0, 0, 1, 1, 2])):
            n = rng.choice([0, 1, 3, 9, 20, 45, 70, 130, 400])
            rid = "q%d" % arrivals
            seqs_a[rid], seqs_b[rid] = make_seq(rid, n, arrivals), make_seq(rid, n, arrivals)
            sa.add(seqs_a[rid])
            sb.add(seqs_b[rid])
            arrivals += 1
        if seqs_a and rng.random() < 0.05:
            rid = rng.choice(list(seqs_a))
            assert (sa.abort(rid) is None) == (sb.abort(rid) is None)
            del seqs_a[rid], seqs_b[rid]
        pa, pb = sa.schedule(), sb.schedule()
        assert plan_as_data(pa) == plan_as_data(pb), step
        assert [s.request_id for s in sa.waiting] == [s.request_id for s in sb.waiting]
        assert [s.request_id for s in sa.running] == [s.request_id for s in sb.running]
        saw["preempted"] += len(pa.preempted)
        saw["ignored"] += len(pa.ignored)
        saw["capped"] += len(pa.capped)
        saw["portions"] += sum(1 for s in pa.scheduled if s.n_tokens > 1 and not s.samples)
        for s in pa.ignored + pa.capped:
            del seqs_a[s.request_id], seqs_b[s.request_id]
        # what the engine does with a plan: the tokens go into the cache, a token is sampled, some requests end
        for plan, cache, sched, seqs in ((pa, ca, sa, seqs_a), (pb, cb, sb, seqs_b)):
            r2 = random.Random(seed * 100000 + step)
            for s in plan.scheduled:
                rid = s.seq.request_id
                if not cache.has_request(rid):
                    cache.add_request(rid)
                assert cache.append(rid, s.n_tokens) == s.start
                cache.commit(rid)
                s.seq.num_computed += s.n_tokens
                if s.samples:
                    s.seq.output_token_ids.append(5)
                    if r2.random() < 0.08 or s.seq.length >= cfg["max_model_len"]:
                        sched.finish(s.seq)
                        del seqs[rid]
            cache.check_invariants()
        for g in range(len(groups)):
            assert ca.num_free_pages(g) == cb.num_free_pages(g)
        for rid in seqs_a:
            assert (seqs_a[rid].state, seqs_a[rid].num_computed, seqs_a[rid].num_preemptions) == \
                   (seqs_b[rid].state, seqs_b[rid].num_computed, seqs_b[rid].num_preemptions)
    assert sa.num_preemptions == sb.num_preemptions
    return saw


@pytest.mark.parametrize("seed", range(12))
def test_scheduler_equals_the_plain_one_over_random_workloads(seed):
    run_workload(seed)


def test_random_workloads_reach_every_decision():
    total = {"preempted": 0, "ignored": 0, "capped": 0, "portions": 0}
    for seed in range(12):
        for k, v in run_workload(seed).items():
            total[k] += v
    assert all(v > 0 for v in total.values()), total


def test_step_metadata_is_what_the_tables_say():
    """The buffer that the library fills for a step against the block tables and slot mappings read one by
    one: positions, segments, state slots, slots, tables (a released page appears as page 0)."""
    m = CacheManager([GroupConfig(4, 32), GroupConfig(2, 32, window=5)], 4)
    rids, lens = ["a", "b", "c"], [9, 1, 3]
    for rid, n in (("a", 6), ("b", 11)):            # a and b hold tokens already
        m.add_request(rid)
        m.append(rid, n)
        m.commit(rid)
    handles, starts, added = m.begin_step(rids, lens)
    assert starts.tolist() == [6, 11, 0] and added.tolist() == [0, 0, 1]
    widths = m.step_widths(handles)
    assert widths == [max(len(m.block_table(r, g)) for r in rids) for g in range(2)]
    N, S, R = sum(lens), 3, 2
    offsets, raw, total = m.step_layout(N, S, R, widths)
    assert all(o % 4 == 0 for o, _ in offsets.values()) and total >= max(o + n for o, n in offsets.values())
    spans = sorted(offsets.values())
    assert all(a[0] + a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    buf = np.full(total, -7, dtype=np.int32)
    m.fill_step(handles, starts, lens, widths, raw, buf)
    sec = lambda name: buf[offsets[name][0]:offsets[name][0] + offsets[name][1]]
    assert sec("positions").tolist() == list(range(6, 15)) + [11] + [0, 1, 2]
    assert sec("seg_of").tolist() == [0] * 9 + [1] + [2] * 3
    assert sec("seg_starts").tolist() == [0, 9, 10, 13] and sec("seg_first").tolist() == [6, 11, 0]
    assert sec("state_slots").tolist() == [m.request(r).state_slot for r in rids]
    assert (sec("token_ids") == -7).all() and (sec("logit_rows") == -7).all()       # the caller's
    for g in range(2):
        want = []
        for rid, st, n in zip(rids, starts.tolist(), lens):
            want += m.slot_mapping(rid, g, st, n)
        assert sec("slots%d" % g).tolist() == want
        tables = sec("tables%d" % g).reshape(S, widths[g])
        for i, rid in enumerate(rids):
            t = m.block_table(rid, g)
            assert tables[i].tolist() == [max(p, 0) for p in t] + [0] * (widths[g] - len(t))
    assert -1 in m.block_table("b", 1)               # the window group did release pages of b
    m.abort_step(rids, handles, added)
    assert not m.has_request("c") and m.num_tokens("a") == 6 and m.request("a").pending == 0
    m.check_invariants()
    # a step that does not fit takes nothing
    before = [m.num_free_pages(g) for g in range(2)]
    with pytest.raises(OutOfPages):
        m.begin_step(["a", "d"], [3, 4 * 40])
    assert [m.num_free_pages(g) for g in range(2)] == before and not m.has_request("d")
    assert m.request("a").pending == 0
    m.check_invariants()
