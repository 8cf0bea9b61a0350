"""Configurations drawn at random (head size in steps of 16, any number of heads and groups, widths,
vocabularies and page sizes that are no powers of two, with and without biases, tied embeddings and rotary
scaling) through the engine, whole, in portions and mixed, in float32 and in bfloat16, against the plain
implementation."""
import os
import random

import pytest
import torch

from helpers import random_tokens, replay_in_process, trace_bulk_then_single, trace_mixed, trace_portions, trace_whole
from plain_llama import plain_llama_forward, read_model_folder
from test_replay_gpu import check

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = random.Random(seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
    nkv = rng.choice([1, 2, 3, 4, 5])
    nh = nkv * rng.choice([1, 2, 3, 4, 7, 8])
    H = rng.choice([64, 80, 96, 128, 192, 264, 520, 1024]) if rng.random() < 0.7 else nh * d
    scaling = None
    if rng.random() < 0.4:
        scaling = dict(rope_type="llama3", factor=rng.choice([2.0, 8.0]), low_freq_factor=1.0, high_freq_factor=4.0,
                       original_max_position_embeddings=64)
    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=rng.choice([97, 256, 331, 1000, 2050]),
               hidden_size=(H + 7) // 8 * 8, intermediate_size=rng.choice([88, 176, 208, 352, 520, 1000, 2048]),
               num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=nh, num_key_value_heads=nkv, head_dim=d,
               rms_norm_eps=rng.choice([1e-5, 1e-6]), rope_theta=rng.choice([10000.0, 500000.0]), rope_scaling=scaling,
               max_position_embeddings=512, tie_word_embeddings=rng.random() < 0.3,
               attention_bias=rng.random() < 0.5, mlp_bias=rng.random() < 0.3, hidden_act="silu", bos_token_id=1,
               eos_token_id=2)
    page = rng.choice([4, 8, 16, 32])
    lens = [rng.choice([1, 2, 5, 17, 40, 77, 130, 200, 300]) for _ in range(5)]
    return cfg, page, lens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [3, 15, 35, 65, 72, 74, 127, 157])
def test_a_configuration_drawn_at_random(tmp_path, seed, dtype):
    cfg_dict, page, lens = draw_config(seed)
    replay_every_way(tmp_path, cfg_dict, page, lens, seed, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,I,V", [(72, 172, 331), (64, 250, 1000), (136, 331, 97), (192, 1004, 2050)])
def test_widths_that_no_kernel_tiles_evenly(tmp_path, H, I, V, dtype):
    """Feed-forward widths that are 4 modulo 8, 2 modulo 4 and odd, with prompts of 17 to 64, 65 to 256 and more rows in
    a step: each number of rows has matrix kernels of its own that ask for multiples of 4 or 8 outputs, and a product
    that none of them takes goes to the library."""
    cfg_dict = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=V, hidden_size=H,
                    intermediate_size=I, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                    rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, max_position_embeddings=512,
                    tie_word_embeddings=False, attention_bias=False, mlp_bias=I % 2 == 0, hidden_act="silu",
                    bos_token_id=1, eos_token_id=2)
    replay_every_way(tmp_path, cfg_dict, 16, [40, 100, 3, 300, 180], H + I, dtype)


def replay_every_way(tmp_path, cfg_dict, page, lens, seed, dtype):
    from lmsf_amd.config import LlamaConfig
    from lmsf_amd.engine import load_engine_core
    from lmsf_amd.weights import write_random_model
    folder = os.path.join(str(tmp_path), "m")
    write_random_model(folder, LlamaConfig.from_dict(dict(cfg_dict, torch_dtype=dtype)), seed=seed, dtype=dtype)
    cfg, w = read_model_folder(folder)
    reqs = {"r%d" % i: random_tokens(n, cfg["vocab_size"], 50 + i) for i, n in enumerate(lens)}
    refs = {rid: plain_llama_forward(cfg, w, toks) for rid, toks in reqs.items()}
    alone = -(-max(lens) // page) + 1
    for what, steps, pages in (("whole", trace_whole(reqs), alone),
                               ("bulk then single", trace_bulk_then_single(reqs, tail=8), alone),
                               ("portions", trace_portions(reqs, seed=seed), alone),
                               ("mixed", trace_mixed(reqs, 512, seed=seed), 512 // page)):
        core = load_engine_core(folder, dtype=dtype, block_size=page, num_pages=pages, max_num_seqs=8)
        got = replay_in_process(core.executor, steps)
        assert all(torch.isfinite(g).all() for g in got.values()), (what, cfg_dict)
        check(got, refs, dtype, "%s, %r, pages of %d" % (what, cfg_dict, page))
        core.storage.manager.check_invariants()
        assert core.storage.manager.num_free_pages(0) == core.storage.groups[0].num_pages
        del core
