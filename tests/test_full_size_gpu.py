"""The engine at the layer sizes of Llama-3-8B (two layers of it, random weights): the shapes that the
kernels are built for, which the tiny configurations never reach: the few-rows products with their fused
epilogues (QKV with rotary embedding and cache write, gate_up with the activation, the LM head over 128,256
columns), the 17-to-64-row products left as partial sums, the library products, the matrix-core attention with
groups of four heads. Compared with the plain implementation on the same bfloat16-stored weights."""
import os

import pytest
import torch

from helpers import random_tokens, replay_in_process, trace_mixed, trace_whole
from lmsf_amd.config import LlamaConfig
from lmsf_amd.weights import write_random_model
from plain_llama import plain_llama_forward, read_model_folder
from test_replay_gpu import check

pytestmark = pytest.mark.gpu

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
    # lengths chosen for the paths: 100 tokens at once (library products), portions of 24 and 40 (17 to 64 rows,
    # partial sums), single tokens of up to four requests together (few rows)
    reqs = {"a": random_tokens(100, V, 1), "b": random_tokens(70, V, 2), "c": random_tokens(41, V, 3),
            "d": random_tokens(9, V, 4)}
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    core = load_engine_core(folder, dtype="bfloat16", block_size=16, num_pages=24, max_num_seqs=8)
    check(replay_in_process(core.executor, trace_whole(reqs)), refs, "bfloat16", "whole")
    steps = trace_mixed(reqs, 24 * 16, seed=3)
    sizes = {len(e["tokens"]) for s in steps for e in s["entries"]}
    rows = {sum(len(e["tokens"]) for e in s["entries"]) for s in steps}
    assert 1 in sizes and any(17 <= r <= 64 for r in rows) and any(r <= 16 for r in rows)
    check(replay_in_process(core.executor, steps), refs, "bfloat16", "mixed")
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == 24
    # greedy tokens of the engine's sampler against the plain logits (ties aside: random weights have none)
    logits = torch.stack([refs[r][-1] for r in reqs])
    assert core.rt.ops.sample(logits.cuda()).tolist() == logits.argmax(dim=-1).tolist()


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
