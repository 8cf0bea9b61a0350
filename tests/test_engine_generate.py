"""Generation through LLMEngine with torch stand-ins for the kernels (CPU): greedy tokens equal the
plain implementation's, preemption by recompute changes nothing, seeded sampling does not depend
on the batch, and the stop rules."""
import pytest

from helpers import TINY, make_model_folder, random_tokens
from plain_llama import plain_greedy_generate, read_model_folder
from torch_ops import TorchOps

from lmsf_amd.engine import EngineArgs, LLMEngine
from lmsf_amd.sampling import SamplingParams


def make_engine(tmp_path, which="A", **kw):
    folder, cfg = make_model_folder(tmp_path, which)
    args = EngineArgs(model=folder, dtype="float32", block_size=TINY[which][2], device="cpu",
                      num_gpu_blocks_override=kw.pop("pages", 64), max_num_seqs=kw.pop("max_num_seqs", 8), **kw)
    return LLMEngine(args, ops=TorchOps()), folder, cfg


def run(engine):
    done = {}
    while engine.has_unfinished_requests():
        for out in engine.step():
            if out.finished:
                done[out.request_id] = out
    return done


def test_greedy_equals_plain(tmp_path):
    engine, folder, cfg = make_engine(tmp_path, "A", prefill_chunk_size=16, max_num_batched_tokens=40)
    cfg_dict, w = read_model_folder(folder)
    prompts = [random_tokens(n, cfg.vocab_size, 10 + n) for n in (1, 7, 33, 64)]
    for i, p in enumerate(prompts):
        engine.add_request(i, p, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))
    done = run(engine)
    for i, p in enumerate(prompts):
        assert done[i].outputs[0].token_ids == plain_greedy_generate(cfg_dict, w, p, 8), i
        assert done[i].outputs[0].finish_reason == "length"
    engine.core.storage.manager.check_invariants()
    assert engine.core.storage.manager.num_free_pages(0) == 64


def test_preemption_reproduces_the_same_tokens(tmp_path):
    """So few pages that requests are preempted and recomputed: greedy and seeded tokens are the same
    as with plenty of pages."""
    results = []
    for pages in (64, 9):
        engine, folder, cfg = make_engine(tmp_path, "A", pages=pages, prefill_chunk_size=16)
        for i, n in enumerate((20, 17, 9)):
            temp = 0.0 if i == 0 else 0.8
            engine.add_request(i, random_tokens(n, cfg.vocab_size, 50 + i),
                               SamplingParams(temperature=temp, max_tokens=20, ignore_eos=True, seed=1234 + i))
        done = run(engine)
        results.append(({i: done[i].outputs[0].token_ids for i in done}, engine.stats["preemptions"]))
        engine.core.storage.manager.check_invariants()
    assert results[1][1] > 0, "the small pool was meant to force a preemption"
    assert results[0][0] == results[1][0]


def test_seeded_sampling_does_not_depend_on_batch(tmp_path):
    engine, folder, cfg = make_engine(tmp_path, "B")
    prompt = random_tokens(12, cfg.vocab_size, 3)
    params = dict(temperature=0.7, top_k=50, top_p=0.9, max_tokens=10, ignore_eos=True, seed=99)
    engine.add_request("alone", prompt, SamplingParams(**params))
    alone = run(engine)["alone"].outputs[0].token_ids
    engine.add_request("x", random_tokens(30, cfg.vocab_size, 4), SamplingParams(temperature=1.0, max_tokens=12))
    engine.add_request("together", prompt, SamplingParams(**params))
    engine.add_request("y", random_tokens(5, cfg.vocab_size, 5), SamplingParams(temperature=0.0, max_tokens=3))
    assert run(engine)["together"].outputs[0].token_ids == alone


def test_stop_rules(tmp_path):
    engine, folder, cfg = make_engine(tmp_path, "A")
    cfg_dict, w = read_model_folder(folder)
    prompt = random_tokens(10, cfg.vocab_size, 8)
    greedy = plain_greedy_generate(cfg_dict, w, prompt, 6)
    # stop_token_ids: stops at the first occurrence, which is kept in the output
    stop_at = greedy[2]
    first = greedy.index(stop_at)
    engine.add_request("s", prompt, SamplingParams(temperature=0.0, max_tokens=6, stop_token_ids=[stop_at],
                                                   ignore_eos=True))
    out = run(engine)["s"].outputs[0]
    assert out.token_ids == greedy[:first + 1] and out.finish_reason == "stop"
    # max_tokens
    engine.add_request("m", prompt, SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True))
    out = run(engine)["m"].outputs[0]
    assert out.token_ids == greedy[:3] and out.finish_reason == "length"
    # EOS (token 2 in config A) ends a request unless ignore_eos
    engine.eos_token_ids = {greedy[1]}
    engine.add_request("e", prompt, SamplingParams(temperature=0.0, max_tokens=6))
    engine.add_request("i", prompt, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    done = run(engine)
    assert done["e"].outputs[0].token_ids == greedy[:greedy.index(greedy[1]) + 1]
    assert done["e"].outputs[0].finish_reason == "stop" and done["i"].outputs[0].token_ids == greedy


def test_context_limit_and_bad_requests(tmp_path):
    engine, folder, cfg = make_engine(tmp_path, "A", max_model_len=32)
    prompt = random_tokens(30, cfg.vocab_size, 2)
    engine.add_request("c", prompt, SamplingParams(temperature=0.0, max_tokens=50, ignore_eos=True))
    out = run(engine)["c"].outputs[0]
    assert len(out.token_ids) == 2 and out.finish_reason == "length"       # 30 + 2 = the context
    engine.add_request("long", random_tokens(33, cfg.vocab_size, 1), SamplingParams(max_tokens=2))
    out = run(engine)["long"]
    assert out.finished and out.outputs[0].token_ids == [] and out.outputs[0].finish_reason == "length"
    with pytest.raises(ValueError):
        engine.add_request("bad", [1, cfg.vocab_size], None)
    with pytest.raises(ValueError):
        engine.add_request("empty", [], None)
    engine.add_request("a", prompt[:5], SamplingParams(max_tokens=50, ignore_eos=True))
    engine.step()
    engine.abort_request("a")
    assert not engine.has_unfinished_requests()
    engine.core.storage.manager.check_invariants()


def test_sampling_params_follow_the_reference():
    for bad in (dict(n=2), dict(best_of=3), dict(use_beam_search=True), dict(temperature=-1.0), dict(top_p=0.0),
                dict(top_p=1.5), dict(top_k=0), dict(top_k=-2), dict(min_p=2.0), dict(max_tokens=0),
                dict(presence_penalty=3.0), dict(frequency_penalty=-3.0), dict(repetition_penalty=2.5),
                dict(stop=[""]), dict(logprobs=1), dict(length_penalty=2.0), dict(early_stopping=True)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    p = SamplingParams(temperature=0.0, top_k=5, top_p=0.5, min_p=0.1)
    assert p.greedy and (p.top_k, p.top_p, p.min_p) == (-1, 1.0, 0.0)
    d = SamplingParams()
    assert (d.temperature, d.top_p, d.top_k, d.max_tokens, d.repetition_penalty) == (1.0, 1.0, -1, 128, 1.0)


@pytest.mark.parametrize("pages", [64, 8])
def test_running_a_step_ahead_changes_no_token(tmp_path, pages):
    """The host launches the next step before it has read the tokens of the one in flight. Requests that end
    on a stop token (found out one step late), by their length limit (known in advance), with penalties (never
    run ahead), requests that arrive under way, an abort, and so few pages that requests are preempted: the
    outputs are those of an engine that reads every step's tokens before it schedules the next."""
    results = []
    for ahead in (False, True):
        engine, folder, cfg = make_engine(tmp_path, "A", pages=pages, prefill_chunk_size=16, run_ahead=ahead)
        V = cfg.vocab_size
        stop_ids = list(range(0, V, 16))          # one token id in sixteen stops a request: they end early
        def add(i, n, **kw):
            engine.add_request(i, random_tokens(n, V, 90 + i), SamplingParams(seed=77 + i, **kw))
        add(0, 20, temperature=0.9, max_tokens=30, stop_token_ids=stop_ids)
        add(1, 17, temperature=0.0, max_tokens=30, ignore_eos=True)
        add(2, 9, temperature=0.7, max_tokens=4, ignore_eos=True, presence_penalty=0.5)
        done, launched_ahead, steps = {}, 0, 0
        while engine.has_unfinished_requests():
            for out in engine.step():
                if out.finished:
                    done[out.request_id] = (out.outputs[0].token_ids, out.outputs[0].finish_reason)
            launched_ahead += engine._inflight is not None
            steps += 1
            if steps == 3:
                add(3, 5, temperature=1.0, max_tokens=18, stop_token_ids=stop_ids)
                add(4, 30, temperature=0.0, max_tokens=20, ignore_eos=True)
            if steps == 9:
                engine.abort_request(4)
        assert (launched_ahead > 5) == ahead
        assert (engine.stats["preemptions"] > 0) == (pages == 8)
        assert set(done) == {0, 1, 2, 3}
        results.append(done)
        engine.core.storage.manager.check_invariants()
        assert engine.core.storage.manager.num_free_pages(0) == pages
    assert results[0] == results[1]
    assert results[0][1][1] == "length" and "stop" in {r[1] for r in results[0].values()}


def test_a_prompt_that_is_too_long_is_ignored_with_a_warning(tmp_path, capsys):
    """A prompt beyond the engine's length limit finishes at once without a token, as in the reference's scheduler
    (core/src/sched/scheduler.rs:368-381), and the engine says so; the request beside it runs as usual."""
    engine, folder, cfg = make_engine(tmp_path, "A", max_model_len=16)
    engine.add_request("long", random_tokens(40, cfg.vocab_size, 1), SamplingParams(temperature=0.0, max_tokens=4))
    engine.add_request("fits", random_tokens(5, cfg.vocab_size, 2), SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    done = run(engine)
    assert done["long"].outputs[0].token_ids == [] and done["long"].outputs[0].finish_reason == "length"
    assert len(done["fits"].outputs[0].token_ids) == 4
    err = capsys.readouterr().err
    assert "'long'" in err and "40 tokens" in err and "too long" in err and "'fits'" not in err


def test_a_step_ahead_that_fails_loses_no_token_and_no_output(tmp_path):
    """The step launched ahead raises (here: the step function refuses it). The step in flight is sound: its tokens
    are appended, its outputs come with the caller's next step(), nothing is counted twice, and the run ends with the
    tokens of an undisturbed run and every page back."""
    from lmsf_amd.engine.executor import StepError
    engine, folder, cfg = make_engine(tmp_path, "A", prefill_chunk_size=16)
    calm, _, _ = make_engine(tmp_path, "A", prefill_chunk_size=16)
    prompts = [random_tokens(n, cfg.vocab_size, 80 + n) for n in (9, 21)]
    for e in (engine, calm):
        for i, p in enumerate(prompts):
            e.add_request(i, p, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    want = {i: o.outputs[0].token_ids for i, o in run(calm).items()}
    real_step, calls, failed = engine.core.executor.step, [0], [0]

    def flaky(entries, prev_tokens=None):
        calls[0] += 1
        if calls[0] in (3, 5):                                   # steps launched ahead of the one in flight
            failed[0] += 1
            raise StepError("refused for the test")
        return real_step(entries, prev_tokens=prev_tokens)

    engine.core.executor.step = flaky
    done, seen = {}, {0: [], 1: [], "too long": []}
    while engine.has_unfinished_requests():
        if calls[0] == 2 and "too long" not in engine._requests and "too long" not in done:
            # a prompt that the scheduler ignores, in the very step whose launch then fails: its output was collected
            # before the failure and must not be lost with it
            engine.add_request("too long", random_tokens(cfg.max_position_embeddings + 5, cfg.vocab_size, 3),
                               SamplingParams(temperature=0.0, max_tokens=2))
        try:
            outs = engine.step()
        except StepError:
            engine.core.storage.manager.check_invariants()
            continue
        for out in outs:
            seen[out.request_id].append(out.outputs[0].latest_token)
            if out.finished:
                done[out.request_id] = out
    assert failed[0] == 2
    assert done.pop("too long").outputs[0].finish_reason == "length" and seen.pop("too long") == [None]
    assert {i: o.outputs[0].token_ids for i, o in done.items()} == want
    # every token of every request was reported exactly once, in order: no output lost, none twice
    assert seen == want
    engine.core.storage.manager.check_invariants()
    assert engine.core.storage.manager.num_free_pages(0) == 64
