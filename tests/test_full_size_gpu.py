"""The engine at the layer sizes of Llama-3-8B (two layers of it, random weights): the shapes that the
kernels are built for, which the tiny configurations never reach: the few-rows products with their fused
epilogues (QKV with rotary embedding and cache write, gate_up with the activation, the LM head over 128,256
columns), the 17-to-64-row products left as partial sums, the library products, the matrix-core attention with
groups of four heads. Compared with the plain implementation on the same bfloat16-stored weights."""
import os

import pytest
import torch

from helpers import (random_tokens, replay_in_process, trace_bulk_then_single, trace_mixed, trace_portions,
                     trace_whole)
from lmsf_amd.config import LlamaConfig
from lmsf_amd.weights import write_random_model
from plain_llama import plain_llama_forward, read_model_folder
from test_replay_gpu import check

pytestmark = pytest.mark.gpu

# At a width of 4,096 the usual N(0, 0.02) weights give the attention scores a spread of 0.02^2 * 4096 = 1.6:
# attention is peaked in both layers, and the rounding of bfloat16 activations costs 1.2 % of the largest logit on
# average and 1.7 % at most over these requests, the same for whole prompts as for every other way of cutting
# (measured; the largest of 128,256 logits' errors). The bound leaves that half as much room again.
BOUND = 2.5e-2

FULL = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=4096,
    intermediate_size=14336, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, rms_norm_eps=1e-5,
    rope_theta=500000.0, rope_scaling=None, max_position_embeddings=8192, tie_word_embeddings=True,
    attention_bias=False, hidden_act="silu", torch_dtype="bfloat16", bos_token_id=128000, eos_token_id=128001)


@pytest.fixture(scope="module")
def full_model(tmp_path_factory):
    folder = os.path.join(str(tmp_path_factory.mktemp("full")), "llama3_8b_layers")
    cfg = LlamaConfig.from_dict(FULL)
    write_random_model(folder, cfg, seed=11, dtype="bfloat16")
    cfg_dict, w = read_model_folder(folder)
    return folder, cfg_dict, w


def test_llama3_8b_layer_sizes_every_product_path(full_model):
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = full_model
    V = cfg["vocab_size"]
    # lengths chosen for the paths: 100 and 70 tokens at once (the 17-and-more-rows and the many-rows products),
    # portions of 24 and 40 (17 to 64 rows, partial sums), single tokens of up to four requests together (few rows)
    reqs = {"a": random_tokens(100, V, 1), "b": random_tokens(70, V, 2), "c": random_tokens(41, V, 3),
            "d": random_tokens(9, V, 4)}
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=24, max_num_seqs=8)
    check(replay_in_process(core.executor, trace_whole(reqs)), refs, "bfloat16", "whole", BOUND)
    steps = trace_mixed(reqs, 24 * 16, seed=3)
    sizes = {len(e["tokens"]) for s in steps for e in s["entries"]}
    rows = {sum(len(e["tokens"]) for e in s["entries"]) for s in steps}
    assert 1 in sizes and any(17 <= r <= 64 for r in rows) and any(r <= 16 for r in rows)
    check(replay_in_process(core.executor, steps), refs, "bfloat16", "mixed", BOUND)
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == 24
    # greedy tokens of the engine's sampler against the plain logits (ties aside: random weights have none)
    logits = torch.stack([refs[r][-1] for r in reqs])
    assert core.rt.ops.sample(logits.cuda()).tolist() == logits.argmax(dim=-1).tolist()


@pytest.mark.parametrize("n_prompt", [200, 300, 700, 2048])
def test_llama3_8b_layer_sizes_whole_prompts_of_hundreds_of_tokens(full_model, n_prompt):
    """Whole prompts of 200 tokens (the many-rows product inside the step program), of 300 and 700 (the BLAS
    library's products called from the program, the many-rows product for down) and of 2,048 (the many-tile prefill
    attention, the tiled rotary and cache kernel, the vectorised activation), then four tokens decoded one by one
    from the cache that the prompt left: the last prompt position and the four after it against the plain
    implementation."""
    from lmsf_amd.engine import StepEntry, load_engine_core
    folder, cfg, w = full_model
    toks = random_tokens(n_prompt + 4, cfg["vocab_size"], 100 + n_prompt)
    ref = plain_llama_forward(cfg, w, toks, last=5)
    core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=-(-(n_prompt + 4) // 16) + 1, max_num_seqs=2,
                            max_num_batched_tokens=2048)
    ex = core.executor
    rows = [ex.step([StepEntry("p", toks[:n_prompt], [n_prompt - 1])]).float().cpu()]
    for t in toks[n_prompt:]:
        rows.append(ex.step([StepEntry("p", [t], [0])]).float().cpu())
    ex.release("p")
    assert ex.program is not None and ex.program_steps >= 2      # (the prompt, then single tokens until their kind is a graph)
    check({"p": torch.cat(rows[:5])}, {"p": ref}, "bfloat16", "a whole prompt of %d tokens and four more" % n_prompt, BOUND)
    core.storage.manager.check_invariants()


def test_llama3_8b_layer_sizes_with_the_library_products_raced_at_load(full_model):
    """``tune_products``: at load the library's candidates race for the products of a full step (1,024 tokens here)
    and of a portion of ``prefill_chunk_size`` tokens on the model's own weights. Prompts of 600 and 1,024 tokens and
    a portion of 512 against the plain implementation."""
    from lmsf_amd.engine import EngineArgs, LLMEngine, StepEntry
    folder, cfg, w = full_model
    engine = LLMEngine(EngineArgs(model=folder, dtype="bfloat16", block_size=16, num_gpu_blocks_override=160,
                                  max_num_seqs=4, max_num_batched_tokens=1024, prefill_chunk_size=512,
                                  tune_products=True, skip_tokenizer_init=True))
    tuned = engine.tuned_products
    assert {m for (m, _n, _k) in tuned} == {512, 1024} and len(tuned) >= 6       # QKV, o, gate_up at either; down stays with this package's product
    assert all(0 < best <= first for first, best in tuned.values())
    ex = engine.core.executor
    reqs = {"a": random_tokens(600, cfg["vocab_size"], 31), "b": random_tokens(1024, cfg["vocab_size"], 32),
            "c": random_tokens(512, cfg["vocab_size"], 33)}
    got = {}
    for rid, toks in reqs.items():
        got[rid] = ex.step([StepEntry(rid, toks, [len(toks) - 2, len(toks) - 1])]).float().cpu()
        ex.release(rid)
    refs = {rid: plain_llama_forward(cfg, w, toks, last=2) for rid, toks in reqs.items()}
    check(got, refs, "bfloat16", "prompts after the race", BOUND)


def test_llama3_8b_layer_sizes_in_true_float32(full_model):
    """The 32-bit path at these sizes (float32 multiply-add products over K = 4,096 and 14,336, the general
    attention kernel), on the same weights: a prompt in two portions and a few single tokens."""
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = full_model
    toks = random_tokens(30, cfg["vocab_size"], 9)
    ref = plain_llama_forward(cfg, w, toks)
    core = load_engine_core(folder, dtype="float32", block_size=16, num_pages=4, max_num_seqs=2)
    parts = [toks[:19], toks[19:26]] + [[t] for t in toks[26:]]
    steps = [{"step": i, "entries": [{"id": "x", "tokens": p, "want": list(range(len(p)))}],
              "end": ["x"] if i == len(parts) - 1 else []} for i, p in enumerate(parts)]
    check(replay_in_process(core.executor, steps), {"x": ref}, "float32", "float32 at full layer sizes")


def test_llama3_8b_layer_sizes_bulk_then_single_and_portions(full_model):
    """The other two ways of cutting at these sizes: most of a request in one step and its last 32 tokens one by
    one (the one-row products with their fused norm, residual and rotary forms), and portions of changing size."""
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = full_model
    V = cfg["vocab_size"]
    reqs = {"a": random_tokens(90, V, 21), "b": random_tokens(37, V, 22)}
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=8, max_num_seqs=4)
    check(replay_in_process(core.executor, trace_bulk_then_single(reqs)), refs, "bfloat16", "bulk then single", BOUND)
    check(replay_in_process(core.executor, trace_portions(reqs, seed=5)), refs, "bfloat16", "portions", BOUND)
    assert core.executor.program is not None and core.executor.program_steps > 8
    core.storage.manager.check_invariants()


def test_llama3_8b_layer_sizes_decode_steps_of_24_40_and_64_requests(full_model):
    """Steps of single tokens of 24, 40 and 64 requests of unequal contexts at these sizes, each kind once
    launched kernel by kernel and captured, then replayed: the 17-and-more-rows products left as partial sums, the
    rotary kernel that adds them up, the attention over the cache with the longest contexts first."""
    from lmsf_amd.engine import StepEntry, load_engine_core
    folder, cfg, w = full_model
    V = cfg["vocab_size"]
    lens = [9 + (61 * i + 3 * i * i) % 109 for i in range(64)]
    assert len(set(lens)) > 30
    reqs = {i: random_tokens(n, V, 500 + i) for i, n in enumerate(lens)}
    tail = 4
    refs = {i: plain_llama_forward(cfg, w, toks, last=tail) for i, toks in reqs.items()}
    core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=sum(-(-n // 16) for n in lens) + 2,
                            max_num_seqs=64)
    ex = core.executor
    for i, toks in reqs.items():
        ex.step([StepEntry(i, toks[:-tail], [])])
    got = {i: [] for i in reqs}

    def decode(ids, k):
        out = ex.step([StepEntry(i, [reqs[i][len(reqs[i]) - tail + k]], [0]) for i in ids]).float().cpu()
        for row, i in zip(out, ids):
            got[i].append(row)

    first, rest = list(range(24)), list(range(24, 64))
    decode(first, 0), decode(rest, 0)            # launched one by one, then captured
    decode(first, 1), decode(rest, 1)            # replayed
    decode(first + rest, 2)                      # 64: launched and captured
    decode(rest + first, 3)                      # replayed, in another order
    kinds = {b for (b, _bucket) in ex._static}
    assert {24, 40, 64} <= kinds and all(sb.graph is not None for sb in ex._static.values())
    check({i: torch.stack(rows) for i, rows in got.items()}, refs, "bfloat16", "decode steps of 24, 40 and 64", BOUND)


def test_loading_leaves_no_holes_in_device_memory():
    """Random weights are made through float32 temporaries twice a tensor's size. Torch keeps freed blocks and
    cuts later allocations out of them: a fused weight made after its first source was read sat in that source's
    freed block with a hole beside it for good (at Llama-3.1-70B widths 101 MB a layer, 8 GB over the model,
    which the cache then lacked). The loader makes the fused buffer first and hands freed blocks back between
    parts. Three layers at those widths: the holes would be 300 MB."""
    import gc
    from lmsf_amd.engine import load_engine_core
    gc.collect()
    torch.cuda.empty_cache()
    base = torch.cuda.memory_reserved() - torch.cuda.memory_allocated()
    cfg = LlamaConfig.from_dict(dict(FULL, hidden_size=8192, num_attention_heads=64, intermediate_size=28672,
                                     num_hidden_layers=3, vocab_size=32000, bos_token_id=1, eos_token_id=2))
    core = load_engine_core(None, config=cfg, dtype="bfloat16", block_size=16, num_pages=8, max_num_seqs=2,
                            load_format="random")
    torch.cuda.empty_cache()
    slack = torch.cuda.memory_reserved() - torch.cuda.memory_allocated() - base
    weights = sum(t.numel() * t.element_size() for p in core.model.parts() for t in p.tensors())
    assert weights > 5e9 and slack < (200 << 20), (slack, weights)


@pytest.mark.parametrize("library", [1, 0])
def test_recorded_program_at_these_sizes_steps_of_300_to_2048_tokens(full_model, library):
    """Steps of 300, 700 and 2,048 tokens (and of 100 beside them) through the program and part by part: the same
    kernels for the same routes, so the same bits. With the BLAS library (its products called from C++ by both) and
    without it (use_library_gemm 0: the deep product of down stays with the many-rows kernel up to 1,024 rows, the
    others fall to the float32 multiply-add kernel; 2,048 tokens are left out there, for the time they would take)."""
    from lmsf_amd.engine import load_engine_core
    from lmsf_amd.ops import get_ops
    folder, cfg, w = full_model
    V = cfg["vocab_size"]
    lens = {"e": 300, "f": 700, "g": 100}
    if library:
        lens["h"] = 2048
    reqs = {r: random_tokens(n, V, 60 + n) for r, n in lens.items()}
    steps = trace_whole(reqs) + trace_portions({"i": random_tokens(900, V, 35)}, seed=4)
    ops = get_ops()
    was = ops.use_library_gemm
    ops.use_library_gemm = library
    try:
        outs = []
        for use_program in (True, False):
            core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=132, max_num_seqs=4,
                                    max_num_batched_tokens=2048, use_program=use_program, enforce_eager=True)
            outs.append(replay_in_process(core.executor, steps))
            if use_program:
                assert core.executor.program_steps >= len(steps)
        for rid in outs[0]:
            assert torch.equal(outs[0][rid], outs[1][rid]), rid
    finally:
        ops.use_library_gemm = was


def test_recorded_program_at_these_sizes_with_the_smallest_workspace(full_model):
    """The step program against the parts at Llama-3-8B widths, bit for bit, with a workspace that starts at
    1 MB and doubles until a step fits: the ring of temporaries then wraps as often as it can, and a buffer
    handed out while its last reader is still to come would show."""
    from lmsf_amd.engine import load_engine_core
    folder, cfg, w = full_model
    V = cfg["vocab_size"]
    reqs = {"a": random_tokens(150, V, 31), "b": random_tokens(60, V, 32), "c": random_tokens(23, V, 33)}
    steps = trace_mixed(reqs, 24 * 16, seed=9) + trace_portions({"d": random_tokens(200, V, 34)}, seed=2)
    outs = []
    for use_program in (True, False):
        core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=24, max_num_seqs=8,
                                use_program=use_program, enforce_eager=True)
        if use_program:
            # (the engine sizes the workspace for its largest step when it is built; here it starts over small)
            core.executor.program_workspace_bytes = 1 << 20
            core.executor.program.workspace = None
            core.executor.program.ensure_workspace(1 << 20)
        outs.append(replay_in_process(core.executor, steps))
        if use_program:
            assert core.executor.program_steps > 30
            grown = core.executor.program.workspace.numel()
            assert (1 << 20) < grown <= (64 << 20), grown
    for rid in outs[0]:
        assert torch.equal(outs[0][rid], outs[1][rid]), rid
