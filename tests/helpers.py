"""Shared by the tests: the two tiny Llama configurations, model folders, traces."""
import json
import os
import random

import torch

from lmsf_amd.config import LlamaConfig, RopeScaling
from lmsf_amd.weights import write_random_model

# Two configurations that differ in every size and option.
TINY_A = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=256, hidden_size=64, intermediate_size=176,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-5, rope_theta=10000.0,
    rope_scaling=None, max_position_embeddings=128, tie_word_embeddings=True, attention_bias=False,
    hidden_act="silu", torch_dtype="float32", bos_token_id=1, eos_token_id=2)
TINY_B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1000, hidden_size=128, intermediate_size=352,
    num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-6,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    max_position_embeddings=512, tie_word_embeddings=False, attention_bias=True, hidden_act="silu",
    torch_dtype="float32", bos_token_id=0, eos_token_id=[7, 9])
# A third one with sizes that are no power of two anywhere (width 80 = 5 heads of 16, vocabulary 331).
TINY_C = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=331, hidden_size=80, intermediate_size=208,
    num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=5, head_dim=48, rms_norm_eps=1e-5,
    rope_theta=1000.0, rope_scaling=None, max_position_embeddings=256, tie_word_embeddings=False,
    attention_bias=False, mlp_bias=True, hidden_act="silu", torch_dtype="float32", bos_token_id=1, eos_token_id=2)

TINY = {"A": (TINY_A, 0, 8), "B": (TINY_B, 1, 16), "C": (TINY_C, 2, 16)}   # config, seed, block size


def make_model_folder(tmp_path, which, dtype="float32", seed=None):
    """Write config.json + model.safetensors of a tiny configuration; returns (folder, config)."""
    cfg_dict, default_seed, _ = TINY[which]
    cfg = LlamaConfig.from_dict(dict(cfg_dict, torch_dtype=dtype))
    folder = os.path.join(str(tmp_path), "tiny_%s_%s" % (which, dtype))
    write_random_model(folder, cfg, seed=default_seed if seed is None else seed, dtype=dtype)
    return folder, cfg


def random_tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]
