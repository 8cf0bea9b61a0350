"""Greedy generation through the entry points on the GPU: the Python one (LLM.generate) and the
command line, in float32 and bfloat16, against the plain implementation."""
import os
import subprocess

import pytest
import torch

from helpers import TINY, make_model_folder, random_tokens
from plain_llama import plain_greedy_generate, plain_llama_forward, read_model_folder

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("which", ["A", "B"])
def test_llm_generate_greedy_float32(tmp_path, which):
    from lmsf_amd import LLM, SamplingParams
    folder, cfg = make_model_folder(tmp_path, which)
    cfg_dict, w = read_model_folder(folder)
    lens = (1, 7, 33, 64) if which == "A" else (3, 40, 150, 300, 17, 90)
    prompts = [random_tokens(n, cfg.vocab_size, 20 + n) for n in lens]
    llm = LLM(model=folder, dtype="float32", block_size=TINY[which][2], num_gpu_blocks_override=96,
              max_num_seqs=8, prefill_chunk_size=64, max_num_batched_tokens=128)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.outputs[0].token_ids == plain_greedy_generate(cfg_dict, w, p, 16), len(p)
    llm.engine.core.storage.manager.check_invariants()


def test_llm_generate_bfloat16_follows_plain_argmax(tmp_path):
    """In bfloat16 a near-tie may flip a token, after which the sequences differ for good; so every
    generated token is checked against the plain logits of the engine's own prefix: it must be the
    argmax or within the bfloat16 error of it."""
    from lmsf_amd import LLM, SamplingParams
    folder, cfg = make_model_folder(tmp_path, "B", dtype="bfloat16")
    cfg_dict, w = read_model_folder(folder)
    prompts = [random_tokens(n, cfg.vocab_size, 40 + n) for n in (5, 70, 200)]
    llm = LLM(model=folder, dtype="bfloat16", block_size=16, num_gpu_blocks_override=64, max_num_seqs=4)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        gen = o.outputs[0].token_ids
        assert len(gen) == 12
        logits = plain_llama_forward(cfg_dict, w, p + gen[:-1])[len(p) - 1:]
        for i, tok in enumerate(gen):
            assert logits[i, tok] >= logits[i].max() - 1.5e-2 * max(0.25, logits[i].abs().max().item()), (len(p), i)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_preemption_on_the_gpu_reproduces_the_same_tokens(tmp_path, dtype):
    """So few pages that running requests are preempted and recomputed, decode steps replayed as graphs in
    between: greedy and seeded tokens are those of a run with plenty of pages. A recomputed request meets other
    batch sizes and portions than before, hence other kernels; the tokens stay the same because the kernels
    that serve one shape of product agree to the bit (and none of these logits is a near-tie)."""
    from lmsf_amd.engine import EngineArgs, LLMEngine
    from lmsf_amd.sampling import SamplingParams
    folder, cfg = make_model_folder(tmp_path, "B", dtype=dtype)
    results = []
    for pages in (96, 12):
        engine = LLMEngine(EngineArgs(model=folder, dtype=dtype, block_size=16, num_gpu_blocks_override=pages,
                                      max_num_seqs=8, prefill_chunk_size=32, max_num_batched_tokens=64))
        for i, n in enumerate((60, 33, 18, 5)):
            engine.add_request(i, random_tokens(n, cfg.vocab_size, 70 + i),
                               SamplingParams(temperature=0.0 if i % 2 == 0 else 0.9, max_tokens=40, ignore_eos=True,
                                              seed=500 + i))
        done = {}
        while engine.has_unfinished_requests():
            for out in engine.step():
                if out.finished:
                    done[out.request_id] = out
        results.append(({i: done[i].outputs[0].token_ids for i in done}, engine.stats["preemptions"]))
        engine.core.storage.manager.check_invariants()
        assert engine.core.storage.manager.num_free_pages(0) == pages
    assert results[1][1] > 0, "the small pool was meant to force a preemption"
    assert results[0][0] == results[1][0]


def test_temperature_sampling_seeded(tmp_path):
    from lmsf_amd import LLM, SamplingParams
    folder, cfg = make_model_folder(tmp_path, "B")
    prompts = [random_tokens(n, cfg.vocab_size, 60 + n) for n in (9, 33)]
    llm = LLM(model=folder, dtype="float32", block_size=16, num_gpu_blocks_override=64, max_num_seqs=4,
              prefill_chunk_size=64)
    sp = SamplingParams(temperature=0.7, max_tokens=24, ignore_eos=True, seed=5)
    a = [o.outputs[0].token_ids for o in llm.generate(prompts, sp)]
    b = [o.outputs[0].token_ids for o in llm.generate(prompts[::-1], sp)][::-1]
    assert a == b and a[0] != a[1]
    c = [o.outputs[0].token_ids for o in llm.generate(prompts, SamplingParams(temperature=0.7, max_tokens=24,
                                                                              ignore_eos=True, seed=6))]
    assert c != a


def test_baseline_configuration_two_sampled_tokens_follow_the_plain_logits(tmp_path):
    """Tiny B in float32, six prompts of 3 to 300 tokens cut into portions of 64 beside the requests that already
    decode, 24 tokens each at temperature 0.7 with seeds: every sampled token is the argmax of the *plain*
    logits of the engine's own prefix, divided by the temperature, plus the noise of (seed, number of the draw,
    vocabulary index)."""
    import numpy as np
    from torch_ops import gumbel_noise
    from lmsf_amd.engine import EngineArgs, LLMEngine
    from lmsf_amd.sampling import SamplingParams
    folder, cfg = make_model_folder(tmp_path, "B")
    cfg_dict, w = read_model_folder(folder)
    V = cfg.vocab_size
    prompts = [random_tokens(n, V, 800 + n) for n in (3, 17, 64, 120, 211, 300)]
    engine = LLMEngine(EngineArgs(model=folder, dtype="float32", block_size=16, num_gpu_blocks_override=128,
                                  max_num_seqs=8, prefill_chunk_size=64, max_num_batched_tokens=96))
    for i, p in enumerate(prompts):
        engine.add_request(i, p, SamplingParams(temperature=0.7, max_tokens=24, ignore_eos=True, seed=900 + i))
    done, mixed_steps = {}, 0
    while engine.has_unfinished_requests():
        for out in engine.step():
            if out.finished:
                done[out.request_id] = out.outputs[0].token_ids
        last = engine.last_step
        mixed_steps += 1 if last["prefill_tokens"] and last["decode_tokens"] else 0
    assert mixed_steps >= 3, "portions of prompts were meant to run beside decoding requests"
    inv_t = np.float32(1.0) / np.float32(0.7)
    for i, p in enumerate(prompts):
        gen = done[i]
        assert len(gen) == 24
        logits = plain_llama_forward(cfg_dict, w, p + gen[:-1])[len(p) - 1:]
        for k, tok in enumerate(gen):
            y = logits[k] * float(inv_t) + gumbel_noise(900 + i, k, V)
            assert int(torch.argmax(y)) == tok or float(y.max() - y[tok]) < 1e-4, (i, k)


def test_command_line(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "A")
    cfg_dict, w = read_model_folder(folder)
    prompt = random_tokens(11, cfg.vocab_size, 9)
    proc = subprocess.run([os.path.join(ROOT, "bin", "lmsf_generate"), "--model", folder, "--dtype", "float32",
                           "--gpu-memory-utilization", "0.5", "--block-size", "8", "--max-model-len", "64",
                           "--prompt-ids", ",".join(map(str, prompt)), "--temperature", "0", "--max-tokens", "8",
                           "--ignore-eos"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = proc.stdout.strip().splitlines()
    assert [int(t) for t in lines[0].split()] == plain_greedy_generate(cfg_dict, w, prompt, 8)
    assert lines[-1].startswith("cost ")


def test_command_line_with_text(tmp_path):
    """The reference's example takes its prompt as text: with a tokenizer.json in the folder the command line
    does too, prints text, and a stop string ends the output."""
    pytest.importorskip("tokenizers")
    from test_text import write_word_tokenizer
    from lmsf_amd.engine.detokenizer import Tokenizer
    folder, cfg = make_model_folder(tmp_path, "A")
    tok = Tokenizer(write_word_tokenizer(folder, n_words=cfg.vocab_size))
    cfg_dict, w = read_model_folder(folder)
    text = "to be or not to be ,"
    want = plain_greedy_generate(cfg_dict, w, tok.encode(text), 8)
    base = [os.path.join(ROOT, "bin", "lmsf_generate"), "--model", folder, "--dtype", "float32",
            "--gpu-memory-utilization", "0.5", "--block-size", "8", "--max-model-len", "64", "--prompt", text,
            "--temperature", "0", "--max-tokens", "8", "--ignore-eos"]
    proc = subprocess.run(base, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = proc.stdout.splitlines()
    assert lines[0] == " " + tok.decode(want) and lines[-1].startswith("cost ")
    stop = tok.decode(want[2:3])
    first = [tok.decode([t]) for t in want].index(stop)
    proc = subprocess.run(base + ["--stop", stop], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.splitlines()[0].split() == tok.decode(want[:first]).split()
    assert ("to gen %d tokens" % (first + 1)) in proc.stdout


@pytest.mark.parametrize("seed", [10011, 10013, 10022, 10036, 10040, 10042])
def test_loads_drawn_at_random_generate_the_plain_tokens(tmp_path, seed):
    """A load drawn at random: which model, how many requests of what lengths, how few pages, the prompt
    portions, the token budget, the live requests allowed, requests that arrive while others run. Greedy in
    float32: every request's tokens are the plain implementation's, however often it was preempted and
    recomputed, and every page comes back. (The seeds are ones whose draw preempts 5 to 26 times.)"""
    import random

    from lmsf_amd.engine import EngineArgs, LLMEngine
    from lmsf_amd.sampling import SamplingParams
    rng = random.Random(seed)
    which = rng.choice(["A", "B", "C"])
    folder, cfg = make_model_folder(tmp_path, which, dtype="float32")
    cfg_dict, w = read_model_folder(folder)
    bs, top = TINY[which][2], cfg.max_position_embeddings
    reqs = []
    for i in range(rng.randint(3, 12)):
        n, mt = rng.choice([1, 2, 5, 9, 17, 30, 47, 64, 90]), rng.choice([1, 2, 5, 12, 25])
        reqs.append((random_tokens(min(n, top - mt - 1), cfg.vocab_size, (seed - 10000) * 100 + i), mt))
    need_one = max(-(-(len(p) + mt) // bs) for p, mt in reqs)
    pages = rng.choice([need_one + 1, need_one + 3, 2 * need_one, 64])
    chunk = rng.choice([None, 8, 16, 32])
    budget = rng.choice([32, 64, 128, 256])
    engine = LLMEngine(EngineArgs(model=folder, dtype="float32", block_size=bs, num_gpu_blocks_override=pages,
                                  max_num_seqs=rng.choice([2, 4, 8, 16]), prefill_chunk_size=chunk,
                                  max_num_batched_tokens=budget, max_model_len=top))
    pending = list(enumerate(reqs))
    rng.shuffle(pending)
    first = rng.randint(1, len(pending))
    add = lambda i, p, mt: engine.add_request(i, p, SamplingParams(temperature=0.0, max_tokens=mt, ignore_eos=True))
    for i, (p, mt) in pending[:first]:
        add(i, p, mt)
    later, done, steps = pending[first:], {}, 0
    while engine.has_unfinished_requests() or later:
        if later and (steps % 3 == 0 or not engine.has_unfinished_requests()):
            i, (p, mt) = later.pop(0)
            add(i, p, mt)
        for out in engine.step():
            if out.finished:
                done[out.request_id] = out
        steps += 1
        assert steps < 5000, "the engine makes no progress"
    engine.core.storage.manager.check_invariants()
    assert engine.core.storage.manager.num_free_pages(0) == pages
    assert engine.stats["preemptions"] >= 5
    for i, (p, mt) in enumerate(reqs):
        assert done[i].outputs[0].token_ids == plain_greedy_generate(cfg_dict, w, p, mt), (i, len(p), mt)
