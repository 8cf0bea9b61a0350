"""The engine against the plain implementation under every way of cutting the work, in float32
and in bfloat16: each request alone and whole; most of it in one step and the last 32 tokens one
by one; portions of changing size; up to four live requests mixed with so few pages that they are
used again; long decoding; the first tokens of a sequence; and the same through bin/trace_run."""
import os

import pytest
import torch

from helpers import (TINY, make_model_folder, random_tokens, replay_in_process, replay_with_program, trace_bulk_then_single,
                     trace_mixed, trace_portions, trace_whole)
from plain_llama import plain_llama_forward, read_model_folder

from lmsf_amd.engine import StepEntry

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def tolerance(dtype, ref, bf16_bound=1.5e-2):
    """float32: rounding of sums of a few hundred terms. bfloat16: activations are rounded to 8 bits of
    mantissa between kernels, a few times per layer; the bound is relative to the largest logit. What the
    rounding costs grows with the spread of the attention scores (std^2 * width of the weights): with the tiny
    configurations' N(0, 0.02) it is 0.3 % of the largest logit."""
    scale = ref.abs().max().item()
    return 3e-5 * max(1.0, scale) if dtype == "float32" else bf16_bound * max(0.25, scale)


def check(got, refs, dtype, what, bf16_bound=1.5e-2):
    for rid, ref in refs.items():
        assert rid in got, (what, rid)
        assert got[rid].shape == ref.shape, (what, rid, got[rid].shape, ref.shape)
        err = (got[rid] - ref).abs()
        t = tolerance(dtype, ref, bf16_bound)
        if err.max().item() > t:
            pos = int(torch.nonzero(err.max(dim=1).values > t)[0])
            raise AssertionError("%s: request %r first differs at position %d (page offset %d): max err %.3g > %.3g"
                                 % (what, rid, pos, pos % 16, err.max().item(), t))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """{(config, storage dtype): (folder, plain config, plain weights)}; bfloat16 models are stored in
    bfloat16, so the plain implementation sees exactly the engine's weights."""
    root = tmp_path_factory.mktemp("models")
    out = {}
    for which in TINY:
        for dtype in ("float32", "bfloat16"):
            folder, _ = make_model_folder(root, which, dtype=dtype)
            cfg, w = read_model_folder(folder)
            out[(which, dtype)] = (folder, cfg, w)
    return out


def requests_for(cfg, which):
    V = cfg["vocab_size"]
    top = cfg["max_position_embeddings"]
    lens = {"A": [1, 7, 33, 64, 128], "B": [3, 45, 130, 300, 77, 260], "C": [2, 100, 255, 31],
            "W": [5, 40, 150, 64, 200]}[which]
    return {"r%d" % i: random_tokens(min(n, top), V, 100 + i) for i, n in enumerate(lens)}


def engine(folder, which, dtype, num_pages, **more):
    from lmsf_amd.engine import load_engine_core
    return load_engine_core(folder, dtype=dtype, block_size=TINY[which][2], num_pages=num_pages, max_num_seqs=8, **more)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "W"])
def test_every_way_of_cutting(models, which, dtype):
    folder, cfg, w = models[(which, dtype)]
    reqs = requests_for(cfg, which)
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    bs = TINY[which][2]
    core = engine(folder, which, dtype, num_pages=-(-max(len(t) for t in reqs.values()) // bs) + 1)
    ex = core.executor
    check(replay_in_process(ex, trace_whole(reqs)), refs, dtype, "whole")
    check(replay_in_process(ex, trace_bulk_then_single(reqs)), refs, dtype, "bulk then single")
    check(replay_in_process(ex, trace_portions(reqs, seed=1)), refs, dtype, "portions")
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == core.storage.groups[0].num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "W"])
def test_mixed_requests_with_page_reuse(models, which, dtype):
    folder, cfg, w = models[(which, dtype)]
    reqs = requests_for(cfg, which)
    reqs.update({"s%d" % i: random_tokens(20 + 9 * i, cfg["vocab_size"], 200 + i) for i in range(4)})
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    longest = -(-max(len(t) for t in reqs.values()) // 64) * 64
    max_tokens = longest + 128            # the longest request and little else: pages must be reused
    steps = trace_mixed(reqs, max_tokens, seed=5)
    assert max(len(s["entries"]) for s in steps) >= 2
    bs = TINY[which][2]
    core = engine(folder, which, dtype, num_pages=max_tokens // bs)
    check(replay_in_process(core.executor, steps), refs, dtype, "mixed")
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == max_tokens // bs


def test_wide_model_leaves_products_unfinished(models, monkeypatch):
    """The wide configuration does reach the kernels that add up partial sums (a step of 40 tokens in
    bfloat16): twice per layer the norm, once per layer the rotation; a step of 8 tokens reaches neither. (Run
    part by part: the recorded program makes the same choices in C++, where this test cannot count them.)"""
    folder, cfg, w = models[("W", "bfloat16")]
    core = engine(folder, "W", "bfloat16", num_pages=8, use_program=False)
    ops = core.executor.rt.ops
    seen = {"norm": 0, "rope": 0}
    norm, rope = ops._add_rms_norm_pending, ops._rope_cache_write_pending

    def count(key, f):
        def g(*a, **k):
            seen[key] += 1
            return f(*a, **k)
        return g
    monkeypatch.setattr(ops, "_add_rms_norm_pending", count("norm", norm))
    monkeypatch.setattr(ops, "_rope_cache_write_pending", count("rope", rope))
    toks = random_tokens(48, cfg["vocab_size"], 77)
    ref = plain_llama_forward(cfg, w, toks)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:40], "want": list(range(40))}], "end": []}]
    got = replay_in_process(core.executor, steps)
    L = cfg["num_hidden_layers"]
    assert seen == {"norm": 2 * L, "rope": L}
    steps = [{"step": 1, "entries": [{"id": "a", "tokens": toks[40:], "want": list(range(8))}], "end": ["a"]}]
    got2 = replay_in_process(core.executor, steps)
    assert seen == {"norm": 2 * L, "rope": L}
    check({"a": torch.cat([got["a"], got2["a"]])}, {"a": ref}, "bfloat16", "wide")
    # the recorded program says what it launched itself: the same choices
    core = engine(folder, "W", "bfloat16", num_pages=8)
    prog = core.executor.program
    core.executor.step([StepEntry("a", toks[:40], list(range(40)))])
    stats = prog.last_step_stats()
    assert stats["norm_over_partials"] == 2 * L and stats["rope_over_partials"] == L and stats["prefill_attention"] == L
    assert stats["mid"] >= 3 * L and "blas" not in stats and "callback" not in stats
    core.executor.step([StepEntry("a", toks[40:], list(range(8)))])
    stats = prog.last_step_stats()
    # (8 rows: the norms run inside the products around them, but for the last, which picks the wanted rows)
    assert "norm_over_partials" not in stats and "rope_over_partials" not in stats and stats["skinny_add_norm"] == 2 * L - 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(models, dtype):
    """One token at a time from the very first token to the end of the context."""
    folder, cfg, w = models[("B", dtype)]
    toks = random_tokens(cfg["max_position_embeddings"], cfg["vocab_size"], 77)
    ref = plain_llama_forward(cfg, w, toks)
    core = engine(folder, "B", dtype, num_pages=len(toks) // 16)
    steps = [{"step": i, "entries": [{"id": "d", "tokens": [t], "want": [0]}], "end": []} for i, t in enumerate(toks)]
    got = replay_in_process(core.executor, steps)
    check(got, {"d": ref}, dtype, "token by token")
    # the first tokens of a sequence alone
    core.executor.release("d")
    got = replay_in_process(core.executor, [{"step": 0, "entries": [{"id": "f", "tokens": toks[:1], "want": [0]}],
                                             "end": ["f"]}])
    check(got, {"f": ref[:1]}, dtype, "first token")


def spike_far_key(folder, cfg, token=5, strength=8.0):
    """A copy of the model folder whose first layer makes every query attend to the key of ``token``:
    the slowest rotary pair of k carries ``strength`` for that token only (k_proj's row there is the
    token's normalised embedding), and every q head carries ``strength`` there through its bias. The
    slowest pair turns by less than a milliradian over the whole context, so the score stays high at
    any distance."""
    import shutil
    from safetensors.torch import load_file, save_file
    from plain_llama import plain_rms_norm
    spiked = folder + "_spiked"
    if os.path.isdir(spiked):
        return spiked
    shutil.copytree(folder, spiked)
    t = load_file(os.path.join(folder, "model.safetensors"))
    H, d, nh = cfg["hidden_size"], cfg["head_dim"], cfg["num_attention_heads"]
    store = t["model.embed_tokens.weight"].dtype
    slow = d // 2 - 1
    h = plain_rms_norm(t["model.embed_tokens.weight"][token].float(), t["model.layers.0.input_layernorm.weight"].float(),
                       cfg["rms_norm_eps"])
    p = "model.layers.0.self_attn."
    wk, bk = t[p + "k_proj.weight"].float(), t[p + "k_proj.bias"].float()
    wq, bq = t[p + "q_proj.weight"].float(), t[p + "q_proj.bias"].float()
    wk[slow] = strength * h / H
    bk[slow] = 0.0
    for head in range(nh):
        wq[head * d + slow] = 0.0
        bq[head * d + slow] = strength
    for name, val in (("k_proj.weight", wk), ("k_proj.bias", bk), ("q_proj.weight", wq), ("q_proj.bias", bq)):
        t[p + name] = val.to(store)
    save_file(t, os.path.join(spiked, "model.safetensors"))
    return spiked


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_key_among_hundreds(models, dtype):
    """Random weights give nearly flat attention, which hides a lost key. Here the weights are made so
    that one token's key stands out, and that token is placed once, early, in a long request: every
    later position's logits depend on reading exactly that far key from its page."""
    folder, cfg, _ = models[("B", dtype)]
    spiked = spike_far_key(folder, cfg)
    cfg, w = read_model_folder(spiked)
    toks = [t if t != 5 else 6 for t in random_tokens(400, cfg["vocab_size"], 31)]
    toks[18] = 5                          # in the second page, far from the end
    ref = plain_llama_forward(cfg, w, toks)
    flat = plain_llama_forward(cfg, w, toks[:18] + [6] + toks[19:])
    assert (ref[300:] - flat[300:]).abs().max() > 10 * tolerance(dtype, ref), "the far key does not matter enough"
    core = engine(spiked, "B", dtype, num_pages=26)
    reqs = {"x": toks}
    check(replay_in_process(core.executor, trace_whole(reqs)), {"x": ref}, dtype, "far key, whole")
    check(replay_in_process(core.executor, trace_bulk_then_single(reqs)), {"x": ref}, dtype, "far key, decode")
    check(replay_in_process(core.executor, trace_portions(reqs, seed=3)), {"x": ref}, dtype, "far key, portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, dtype, tmp_path):
    """The same comparison through the replay program, as a user runs it."""
    folder, cfg, w = models[("B", dtype)]
    reqs = requests_for(cfg, "B")
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    max_tokens = 320 + 128
    steps = trace_mixed(reqs, max_tokens, seed=11)
    # some steps want nothing, and one request wants only a few places
    steps[0]["entries"][0]["want"] = []
    got = replay_with_program(TRACE_RUN, folder, dtype, steps, str(tmp_path / "out"), max_tokens, cfg["vocab_size"])
    first = steps[0]["entries"][0]
    refs_cut = dict(refs)
    refs_cut[first["id"]] = refs[first["id"]][len(first["tokens"]):]
    check(got, refs_cut, dtype, "trace_run mixed")


def test_trace_run_with_another_page_size(models, tmp_path):
    """Tiny A at its own page size of 8 through the program (--block-size), with so few pages that they are
    used again."""
    folder, cfg, w = models[("A", "float32")]
    reqs = requests_for(cfg, "A")
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    max_tokens = 128 + 128
    steps = trace_mixed(reqs, max_tokens, seed=3)
    got = replay_with_program(TRACE_RUN, folder, "float32", steps, str(tmp_path / "out"), max_tokens, cfg["vocab_size"],
                              extra_args=["--block-size", "8"])
    check(got, refs, "float32", "trace_run, pages of 8")


def test_trace_run_with_random_weights(tmp_path):
    """--random CONFIG.json --seed: the same seed gives the same logits, another seed others, and cutting the
    tokens differently changes nothing."""
    import json
    import numpy as np
    from helpers import TINY
    cfg = TINY["B"][0]
    path = tmp_path / "cfg.json"
    path.write_text(json.dumps(cfg))
    toks = random_tokens(40, cfg["vocab_size"], 9)
    whole = [{"step": 0, "entries": [{"id": "a", "tokens": toks, "want": [38, 39]}], "end": ["a"]}]
    cut = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:17], "want": []}], "end": []},
           {"step": 1, "entries": [{"id": "a", "tokens": toks[17:39], "want": [21]}], "end": []},
           {"step": 2, "entries": [{"id": "a", "tokens": toks[39:], "want": [0]}], "end": ["a"]}]

    def run(steps, seed, name):
        return replay_with_program(TRACE_RUN, None, "float32", steps, str(tmp_path / name), 64, cfg["vocab_size"],
                                   extra_args=["--random", str(path), "--seed", str(seed), "--num-gpu-blocks", "5"])["a"]
    a, b, c = run(whole, 1, "a"), run(cut, 1, "b"), run(whole, 2, "c")
    assert torch.allclose(a, b, atol=3e-5) and not torch.allclose(a, c, atol=1e-3)
    assert np.isfinite(a.numpy()).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_equals_eager(models, dtype):
    """Decode steps are captured as HIP graphs and replayed. Every replay must give what the same step
    gives kernel by kernel: the comparison is bitwise, over many replays, with eager steps of other
    shapes (prompt portions) and synchronisations between the replays."""
    folder, cfg, w = models[("B", dtype)]
    from lmsf_amd.engine import load_engine_core
    reqs = {"p": random_tokens(70, cfg["vocab_size"], 301), "q": random_tokens(45, cfg["vocab_size"], 302),
            "r": random_tokens(33, cfg["vocab_size"], 303)}
    steps = trace_mixed(reqs, 512, seed=21, prompt_fraction=0.3)
    assert sum(1 for s in steps if all(len(e["tokens"]) == 1 for e in s["entries"])) > 40
    outs = []
    for eager in (True, False):
        core = load_engine_core(folder, dtype=dtype, block_size=16, num_pages=32, max_num_seqs=8,
                                enforce_eager=eager)
        assert core.executor.use_graphs == (not eager)
        outs.append(replay_in_process(core.executor, steps))
        if not eager:
            assert core.executor._static and all(sb.graph is not None for sb in core.executor._static.values())
    for rid in reqs:
        assert torch.equal(outs[0][rid], outs[1][rid]), rid


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_many_requests_of_different_lengths(models, dtype):
    """Twenty requests of 3 to 250 tokens: each prompt whole but for its last six tokens, then six steps that
    decode all twenty at once, captured and replayed. From sixteen requests on the attention over the cache
    takes the requests with the longest contexts first, in an order that changes from step to step; the logits
    are the plain implementation's whatever the order."""
    folder, cfg, w = models[("B", dtype)]
    from lmsf_amd.engine import load_engine_core
    V = cfg["vocab_size"]
    lens = [3 + (37 * i * i + 11 * i) % 248 for i in range(20)]
    assert len(set(lens)) > 15 and max(lens) > 200 and min(lens) < 12
    reqs = {"m%d" % i: random_tokens(max(n, 8), V, 400 + i) for i, n in enumerate(lens)}
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    steps, n_step = [], 0
    for rid, toks in reqs.items():
        n = len(toks) - 6
        steps.append({"step": n_step, "entries": [{"id": rid, "tokens": toks[:n], "want": list(range(n))}], "end": []})
        n_step += 1
    for k in range(6, 0, -1):
        # the lengths' order changes under way: every second request is left out of the third step
        ids = [rid for i, rid in enumerate(reqs) if not (k == 4 and i % 2)]
        steps.append({"step": n_step, "entries": [{"id": rid, "tokens": [reqs[rid][len(reqs[rid]) - k - (1 if k <= 4 and int(rid[1:]) % 2 else 0)]],
                                                   "want": [0]} for rid in ids], "end": []})
        n_step += 1
    # the requests left out once are one token behind: one more step for them
    late = [rid for i, rid in enumerate(reqs) if i % 2]
    steps.append({"step": n_step, "entries": [{"id": rid, "tokens": [reqs[rid][-1]], "want": [0]} for rid in late],
                  "end": list(reqs)})
    core = load_engine_core(folder, dtype=dtype, block_size=16, num_pages=sum(-(-len(t) // 16) for t in reqs.values()) + 2,
                            max_num_seqs=32)
    got = replay_in_process(core.executor, steps)
    assert any(b >= 16 for (b, _bucket) in core.executor._static), "no decode step of sixteen or more was captured"
    check(got, refs, dtype, "twenty requests")
    core.storage.manager.check_invariants()


@pytest.mark.parametrize("keep", [False, True])
def test_float32_checkpoint_in_a_bfloat16_run(models, keep):
    """A checkpoint stored in 32 bits in a bfloat16 run: its matrices are cast to bfloat16 at load, as the reference
    casts (core/src/model_executor/models/model_factory.rs:124-139); the norms' weights keep their 32 bits. On
    request (keep_float32_weights) the matrices stay as stored, with a warning: activations and cache are bfloat16,
    the products run in float32 arithmetic. Either way the logits are the plain implementation's within the
    bfloat16 bound, under portions and single tokens alike."""
    import warnings
    folder, cfg, w = models[("B", "float32")]
    from lmsf_amd.engine import load_engine_core
    if keep:
        with pytest.warns(UserWarning, match="stored in 32 bits"):
            core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=24, max_num_seqs=4,
                                    keep_float32_weights=True)
    else:
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=24, max_num_seqs=4)
    for part in core.model.parts():
        wt = getattr(part, "weight", None)
        if wt is not None and wt.dim() == 2:
            assert wt.dtype == (torch.float32 if keep else torch.bfloat16), part.prefix
    assert core.model.final_norm.weight.dtype == torch.float32
    assert core.model.bindings[0].k_pages.dtype == torch.bfloat16
    reqs = {"a": random_tokens(150, cfg["vocab_size"], 31), "b": random_tokens(40, cfg["vocab_size"], 32)}
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    check(replay_in_process(core.executor, trace_bulk_then_single(reqs)), refs, "bfloat16", "float32 weights, bulk then single")
    check(replay_in_process(core.executor, trace_portions(reqs, seed=4)), refs, "bfloat16", "float32 weights, portions")


def test_page_count_ignores_memory_that_torch_only_caches(models):
    """Sizing the cache after a large tensor was freed: torch keeps the block, the page count must not."""
    folder, cfg, w = models[("B", "bfloat16")]
    from lmsf_amd.cache.storage import plan_groups
    from lmsf_amd.engine import load_engine_core
    from lmsf_amd.engine.core import profile_num_pages
    core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=4, max_num_seqs=4)
    big = torch.empty(24 << 30, dtype=torch.uint8, device="cuda:0")
    del big
    assert torch.cuda.memory_reserved() - torch.cuda.memory_allocated() > 20 << 30
    seqs = 1 << 18
    n = profile_num_pages(core.model, core.rt, 16, 0.5, 2048, seqs, 4096)[0]
    free, total = torch.cuda.mem_get_info()
    groups, _ = plan_groups(core.model.cache_requirements(), 16)
    act = 2048 * (128 * 4 * 2 + 704 * 2 * 3) + seqs * 1000 * 4 * 3 + (512 << 20)
    want = (int(total * 0.5) - (total - free) - act) / groups[0].bytes_per_page(2)
    assert abs(n - want) / want < 0.02, (n, want)
    assert torch.cuda.memory_reserved() - torch.cuda.memory_allocated() < 1 << 30


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "W"])
def test_recorded_program_gives_the_bits_of_the_parts(models, which, dtype):
    """The model's kernel calls recorded once and run from C++ (one call a step) against the same model run
    part by part from Python: the same kernels with the same arguments, so the logits are equal bit for bit,
    under portions, mixed steps with page reuse and single tokens."""
    folder, cfg, w = models[(which, dtype)]
    from lmsf_amd.engine import load_engine_core
    reqs = requests_for(cfg, which)
    longest = -(-max(len(t) for t in reqs.values()) // 64) * 64
    traces = [trace_portions(reqs, seed=2), trace_mixed(reqs, longest + 128, seed=8), trace_bulk_then_single(reqs)]
    bs = TINY[which][2]
    outs = []
    for use_program in (True, False):
        core = load_engine_core(folder, dtype=dtype, block_size=bs, num_pages=(longest + 128) // bs, max_num_seqs=8,
                                use_program=use_program, enforce_eager=True)
        assert (core.executor.program is not None) == use_program
        outs.append([replay_in_process(core.executor, steps) for steps in traces])
        if use_program:
            assert core.executor.program_steps > 20
    for a, b in zip(*outs):
        for rid in reqs:
            assert torch.equal(a[rid], b[rid]), rid
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    check(outs[0][1], refs, dtype, "recorded program, mixed")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_any_part_may_run_in_python_inside_the_program(models, dtype):
    """The program's callback operation with Llama's own parts: one kind of part after the other is made to run in
    Python in the middle of the recorded program (its operands are then finished tensors in the workspace, what it
    returns is copied to its place), the rest stays native. In float32 every variant gives the bits of the model run
    part by part; in bfloat16 a part that runs in Python takes finished tensors where its native form takes the
    unfinished products of its neighbours (other kernels, other roundings), so there the plain implementation is
    the yardstick. Under mixed steps with page reuse."""
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = models[("B", dtype)]
    reqs = requests_for(cfg, "B")
    longest = -(-max(len(t) for t in reqs.values()) // 64) * 64
    steps = trace_mixed(reqs, longest + 128, seed=11)
    bs = TINY["B"][2]

    def run(python_parts):
        core = load_engine_core(folder, dtype=dtype, block_size=bs, num_pages=(longest + 128) // bs, max_num_seqs=8,
                                use_program=python_parts is not None, enforce_eager=True)
        if python_parts:
            core.executor.python_parts = python_parts
            core.executor._record_program()
            assert len(core.executor.program.callbacks) > 0
        return replay_in_process(core.executor, steps), core.executor.program_steps

    want, _ = run(None)
    kinds = {"block": lambda p, n: type(p).__name__ == "PreNormResidualBlock" and p.prefix.endswith(".1"),
             "mixer": lambda p, n: type(p).__name__ == "PagedAttention",
             "feed-forward": lambda p, n: type(p).__name__ == "GatedMLP",
             "norms": lambda p, n: type(p).__name__ == "RMSNorm" and n == "forward_add",
             "embedding and head": lambda p, n: type(p).__name__ in ("TokenEmbedding", "LMHead"),
             "a layer's linear parts": lambda p, n: type(p).__name__ in ("Linear", "FusedLinear") and ".layers.0." in p.prefix}
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    for name, pred in kinds.items():
        got, steps_run = run(pred)
        assert steps_run >= len(steps), name
        if dtype == "float32":
            for rid in reqs:
                assert torch.equal(got[rid], want[rid]), (name, rid)
        check(got, refs, dtype, "in Python: " + name)


def test_a_switch_point_moved_between_two_mixed_steps(models):
    """Somebody moves one of the kernels' switch points between two steps that hold a prompt's portion beside single
    tokens: the program is recorded again before anything of the next step is built, and that step's attention
    plan belongs to it (the plan's layout travels with the step, not with the program object). Against the model
    run part by part under the same settings, bit for bit."""
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = models[("B", "bfloat16")]
    V = cfg["vocab_size"]
    toks = {r: random_tokens(70, V, 90 + i) for i, r in enumerate("abc")}

    def run(use_program):
        core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=24, max_num_seqs=4,
                                use_program=use_program, enforce_eager=True)
        ex, ops, outs = core.executor, core.rt.ops, []
        was = ops.skinny_max_rows
        try:
            ex.step([StepEntry("a", toks["a"][:30], []), StepEntry("b", toks["b"][:50], [])])
            first = ex.program
            outs.append(ex.step([StepEntry("a", toks["a"][30:31], [0]), StepEntry("b", toks["b"][50:51], [0]),
                                 StepEntry("c", toks["c"][:40], [39])]))
            ops.skinny_max_rows = 8                       # 9 to 16 rows now go to the 17-and-more-rows kernel
            outs.append(ex.step([StepEntry("a", toks["a"][31:32], [0]), StepEntry("b", toks["b"][51:52], [0]),
                                 StepEntry("c", toks["c"][40:50], [9])]))
            if use_program:
                assert ex.program is not first and ex.program is not None
        finally:
            ops.skinny_max_rows = was
        return [o.float().cpu() for o in outs]

    a, b = run(True), run(False)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    ref = plain_llama_forward(cfg, w, toks["c"][:50])
    check({"c": torch.stack([a[0][2], a[1][2]])}, {"c": ref[[39, 49]]}, "bfloat16", "after a switch point moved")


@pytest.mark.parametrize("which", ["A", "B", "C", "W"])
def test_bfloat16_with_peaked_attention_in_every_layer(tmp_path, which):
    """Weights several times larger than the usual N(0, 0.02): the scores of every layer get a spread (their
    standard deviation is about std^2 * width, here 0.4) and every query leans on some keys more than on others.
    Measured at these sizes: changing one far token of a prompt then moves the last position's logits by 8 to
    30 % of the largest logit, while bfloat16 rounding costs under 1 % (it grows with the same spread: 2 to 4 %
    at a spread of 2.5, which is why the weights are not larger still). So a key read from a wrong page or slot,
    in any layer, is an order of magnitude beyond the bound. All four ways of cutting."""
    import math
    width = TINY[which][0]["hidden_size"]
    folder, cfg_obj = make_model_folder(tmp_path, which, dtype="bfloat16", std=math.sqrt(0.4 / width))
    cfg, w = read_model_folder(folder)
    reqs = requests_for(cfg, which)
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    longest = -(-max(len(t) for t in reqs.values()) // 64) * 64
    bs = TINY[which][2]
    core = engine(folder, which, "bfloat16", num_pages=(longest + 128) // bs)
    check(replay_in_process(core.executor, trace_whole(reqs)), refs, "bfloat16", "peaked, whole")
    check(replay_in_process(core.executor, trace_bulk_then_single(reqs)), refs, "bfloat16", "peaked, bulk then single")
    check(replay_in_process(core.executor, trace_portions(reqs, seed=3)), refs, "bfloat16", "peaked, portions")
    check(replay_in_process(core.executor, trace_mixed(reqs, longest + 128, seed=6)), refs, "bfloat16", "peaked, mixed")
    core.storage.manager.check_invariants()
