"""The scheduler's decisions, with the real cache manager and no model: FCFS, the token budget,
portions, admission with a watermark, and what happens when pages run out."""
import random

import pytest

from lmsf_amd.cache import CacheManager, GroupConfig
from lmsf_amd.engine.scheduler import Scheduler, SchedulerConfig
from lmsf_amd.engine.sequence import Sequence, SequenceState
from lmsf_amd.sampling import SamplingParams


def make(num_pages=16, page_size=4, budget=32, max_seqs=8, chunk=None, max_len=64, watermark=0.0):
    cache = CacheManager([GroupConfig(page_size, num_pages)], num_state_slots=max_seqs)
    return Scheduler(SchedulerConfig(budget, max_seqs, max_len, chunk, watermark), cache), cache


def seq(rid, n_prompt, arrival, max_tokens=100):
    return Sequence(rid, list(range(1, n_prompt + 1)), SamplingParams(max_tokens=max_tokens, temperature=0.0),
                    arrival, seed=0)


def run_plan(sched, cache, plan, token=7):
    """Do what the engine does after schedule(): take the pages, advance, sample a token."""
    for s in plan.scheduled:
        if not cache.has_request(s.seq.request_id):
            cache.add_request(s.seq.request_id)
        assert cache.append(s.seq.request_id, s.n_tokens) == s.start
        cache.commit(s.seq.request_id)
        s.seq.num_computed += s.n_tokens
        if s.samples:
            s.seq.output_token_ids.append(token)
    cache.check_invariants()


def test_fcfs_and_budget():
    sched, cache = make(num_pages=64, budget=20)
    a, b, c = seq("a", 12, 0), seq("b", 12, 1), seq("c", 3, 2)
    for s in (a, b, c):
        sched.add(s)
    plan = sched.schedule()
    # a whole, then what is left of the budget for b; c has to wait its turn behind b
    assert [(s.seq.request_id, s.start, s.n_tokens, s.samples) for s in plan.scheduled] == \
        [("a", 0, 12, True), ("b", 0, 8, False)]
    assert plan.num_tokens <= 20
    run_plan(sched, cache, plan)
    plan = sched.schedule()
    # a decodes one token, b finishes its prompt, c is admitted with the rest
    assert [(s.seq.request_id, s.start, s.n_tokens, s.samples) for s in plan.scheduled] == \
        [("a", 12, 1, True), ("b", 8, 4, True), ("c", 0, 3, True)]


def test_prefill_chunk_size():
    sched, cache = make(num_pages=64, budget=16, chunk=5)
    a = seq("a", 11, 0)
    sched.add(a)
    sizes = []
    for _ in range(3):
        plan = sched.schedule()
        sizes.append([(s.start, s.n_tokens, s.samples) for s in plan.scheduled])
        run_plan(sched, cache, plan)
    assert sizes == [[(0, 5, False)], [(5, 5, False)], [(10, 1, True)]]
    sched.add(seq("b", 9, 1))
    plan = sched.schedule()
    assert [(s.seq.request_id, s.n_tokens) for s in plan.scheduled] == [("a", 1), ("b", 5)]


def test_decoding_requests_get_their_token_before_prompt_portions():
    """An earlier arrival in the middle of a long prompt, a portion size of the whole budget, and a later
    request that decodes: the decoder gets its token in every step and the prompt the rest."""
    sched, cache = make(num_pages=64, budget=8, chunk=8, max_len=128)
    sched.add(seq("short", 3, 1))
    run_plan(sched, cache, sched.schedule())                  # short's prompt: it decodes from now on
    long = seq("long", 40, 0)                                 # an earlier arrival number than short's
    sched.add(long)
    for step in range(5):
        plan = sched.schedule()
        got = [(s.seq.request_id, s.n_tokens) for s in plan.scheduled]
        assert got == [("short", 1), ("long", 7)], (step, got)
        assert plan.num_tokens <= 8
        run_plan(sched, cache, plan)
    assert long.num_computed == 35


def test_a_decoder_without_pages_yields_to_an_earlier_prompt_and_a_prompt_without_pages_waits():
    sched, cache = make(num_pages=4, page_size=4, budget=16, max_len=64)
    old, new = seq("old", 12, 0), seq("new", 4, 1)
    sched.add(old)
    sched.add(new)
    plan = sched.schedule()
    assert [(s.seq.request_id, s.n_tokens) for s in plan.scheduled] == [("old", 12), ("new", 4)]
    run_plan(sched, cache, plan)                              # all 4 pages are full
    plan = sched.schedule()
    # both decode and neither has a page: the later arrival gives its page up, the earlier takes it
    assert [x.request_id for x in plan.preempted] == ["new"]
    assert [(s.seq.request_id, s.n_tokens) for s in plan.scheduled] == [("old", 1)]
    run_plan(sched, cache, plan)
    cache.check_invariants()

    # a prompt in its middle that finds no page while a later arrival decodes on its own page's slack keeps
    # what it holds and sits the step out
    sched, cache = make(num_pages=4, page_size=4, budget=7, chunk=6, max_len=64)
    dec = seq("dec", 1, 1)
    sched.add(dec)
    run_plan(sched, cache, sched.schedule())                  # dec holds one page with one token
    pro = seq("pro", 16, 0)
    sched.add(pro)
    for _ in range(2):                                        # 1 + 6 tokens a step: pro takes the other 3 pages
        plan = sched.schedule()
        run_plan(sched, cache, plan)
    assert pro.num_computed == 12 and cache.num_free_pages(0) == 0
    plan = sched.schedule()
    assert [(s.seq.request_id, s.n_tokens) for s in plan.scheduled] == [("dec", 1)] and not plan.preempted
    run_plan(sched, cache, plan)
    assert cache.tokens_held(["pro"]).tolist() == [12]
    # dec's page is full now: it is the latest arrival, so it yields, and pro goes on with its page
    plan = sched.schedule()
    assert [x.request_id for x in plan.preempted] == ["dec"]
    assert [(s.seq.request_id, s.start, s.n_tokens) for s in plan.scheduled] == [("pro", 12, 4)]


def test_too_long_prompt_is_ignored():
    sched, cache = make(max_len=10)
    s = seq("long", 11, 0)
    sched.add(s)
    sched.add(seq("ok", 4, 1))
    plan = sched.schedule()
    assert [x.request_id for x in plan.ignored] == ["long"] and s.state == SequenceState.FINISHED_IGNORED
    assert s.state.finish_reason == "length"
    assert [x.seq.request_id for x in plan.scheduled] == ["ok"]


def test_admission_waits_for_pages_above_watermark():
    sched, cache = make(num_pages=10, page_size=4, budget=64, watermark=0.2)   # 2 pages kept free
    sched.add(seq("a", 24, 0))      # 6 pages
    plan = sched.schedule()
    run_plan(sched, cache, plan)
    sched.add(seq("b", 12, 1))      # 3 pages: 4 free - 3 < 2
    plan = sched.schedule()
    assert [s.seq.request_id for s in plan.scheduled] == ["a"]
    assert len(sched.waiting) == 1 and not plan.preempted


def test_running_out_of_pages_preempts_latest_arrival():
    sched, cache = make(num_pages=6, page_size=4, budget=64)
    a, b = seq("a", 11, 0), seq("b", 8, 1)
    sched.add(a)
    sched.add(b)
    plan = sched.schedule()
    run_plan(sched, cache, plan)                      # a: 3 pages (11), b: 2 pages (8); 1 free
    plan = sched.schedule()                           # a -> 12 fits its page; b -> 9 takes the last page
    run_plan(sched, cache, plan)
    assert cache.num_free_pages() == 0
    plan = sched.schedule()                           # a -> 13 needs a page: b, the latest arrival, gives way
    assert [s.seq.request_id for s in plan.scheduled] == ["a"]
    assert [s.request_id for s in plan.preempted] == ["b"]
    assert b.state == SequenceState.WAITING and b.num_computed == 0 and sched.waiting[0] is b
    assert not cache.has_request("b")
    run_plan(sched, cache, plan)
    # b comes back from the front of the queue and recomputes its prompt and the tokens it had generated
    plan = sched.schedule()
    ids = {s.seq.request_id: (s.start, s.n_tokens, s.samples) for s in plan.scheduled}
    assert ids["a"][1] == 1
    if "b" in ids:
        assert ids["b"][0] == 0 and ids["b"][1] <= b.length


def test_alone_and_out_of_pages_is_capped():
    sched, cache = make(num_pages=2, page_size=4, budget=64, max_len=64)
    a = seq("a", 7, 0)
    sched.add(a)
    plan = sched.schedule()
    run_plan(sched, cache, plan)                      # 8 tokens after the sampled one is fed
    plan = sched.schedule()
    run_plan(sched, cache, plan)
    plan = sched.schedule()                           # token 9 needs a third page
    assert [s.request_id for s in plan.capped] == ["a"] and a.state == SequenceState.FINISHED_LENGTH_CAPPED
    assert not cache.has_request("a") and cache.num_free_pages() == 2
    assert not sched.has_unfinished()


def test_prompt_larger_than_pool_is_ignored():
    sched, cache = make(num_pages=2, page_size=4, max_len=64)
    sched.add(seq("big", 9, 0))
    plan = sched.schedule()
    assert [s.request_id for s in plan.ignored] == ["big"]


def test_abort_in_either_queue():
    sched, cache = make()
    a, b = seq("a", 5, 0), seq("b", 5, 1)
    sched.add(a)
    run_plan(sched, cache, sched.schedule())
    sched.add(b)
    assert sched.abort("b") is b and b.state == SequenceState.FINISHED_ABORTED
    assert sched.abort("a") is a and not cache.has_request("a")
    assert sched.abort("nobody") is None
    cache.check_invariants()
    assert cache.num_free_pages() == 16 and not sched.has_unfinished()


def test_max_num_seqs():
    sched, cache = make(num_pages=64, max_seqs=2, budget=64)
    for i in range(4):
        sched.add(seq(i, 3, i))
    plan = sched.schedule()
    assert [s.seq.request_id for s in plan.scheduled] == [0, 1]


@pytest.mark.parametrize("seed", range(6))
def test_random_load_keeps_invariants(seed):
    """Random arrivals, lengths and finishes on a small pool: the budget is never exceeded, pages are
    never lost or held twice, every request ends, and at the end every page is free."""
    rng = random.Random(seed)
    sched, cache = make(num_pages=24, page_size=4, budget=24, max_seqs=5, chunk=rng.choice([None, 7]),
                        max_len=60, watermark=0.05)
    pending = [seq(i, rng.randint(1, 40), i, max_tokens=rng.randint(1, 30)) for i in range(30)]
    done, arrivals = [], 0
    for step in range(5000):
        while pending and rng.random() < 0.4:
            sched.add(pending.pop(0))
        if not sched.has_unfinished():
            if not pending:
                break
            continue
        plan = sched.schedule()
        assert plan.num_tokens <= 24
        assert len({s.seq.request_id for s in plan.scheduled}) == len(plan.scheduled)
        for s in plan.scheduled:
            assert s.start == s.seq.num_computed and s.n_tokens >= 1
        run_plan(sched, cache, plan)
        done += plan.ignored + plan.capped
        for s in plan.scheduled:
            q = s.seq
            if s.samples and (len(q.output_token_ids) >= q.params.max_tokens or q.length >= 60):
                q.state = SequenceState.FINISHED_LENGTH_CAPPED
                sched.finish(q)
                done.append(q)
    assert len(done) == 30 and not sched.has_unfinished()
    cache.check_invariants()
    assert cache.num_free_pages() == 24 and cache.num_free_state_slots() == 5


def test_a_request_may_finish_while_it_waits():
    """A request preempted after its last token was sampled ends in the waiting queue: the engine finishes it
    there, and the queue must not keep it."""
    sched, cache = make(num_pages=4, page_size=4, budget=16, max_len=64)
    old, new = seq("old", 12, 0), seq("new", 4, 1)
    sched.add(old)
    sched.add(new)
    run_plan(sched, cache, sched.schedule())
    plan = sched.schedule()                                   # no page for both: "new" goes back to waiting
    assert [x.request_id for x in plan.preempted] == ["new"]
    run_plan(sched, cache, plan)
    sched.finish(new)                                         # ... and turns out to have ended with its last token
    assert [s.request_id for s in sched.waiting] == [] and sched.has_unfinished()
    for _ in range(3):
        plan = sched.schedule()
        assert [(s.seq.request_id, s.n_tokens) for s in plan.scheduled] == [("old", 1)]
        run_plan(sched, cache, plan)
    cache.check_invariants()
