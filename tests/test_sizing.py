"""Decisions made before the first step that need no GPU: page counts, the replay program's pool, head sizes
that no kernel takes, the float16 warning."""
import pytest
import torch

from lmsf_amd.cache.storage import GroupLayout
from lmsf_amd.config import LlamaConfig
from lmsf_amd.engine.core import pages_for_budget, resolve_dtype
from lmsf_amd.entrypoints.replay import pages_for
from lmsf_amd.parts.base import CacheSpec


def test_page_count_follows_the_bytes_that_are_left():
    # Llama-3.1-70B shape on a 288 GiB card: 80 layers, 8 kv heads of 128, pages of 16 tokens, bfloat16
    groups = [GroupLayout(CacheSpec(8, 128, None), list(range(80)), 16)]
    per_page = 80 * 2 * 8 * 16 * 128 * 2
    assert groups[0].bytes_per_page(2) == per_page
    total, weights, act = 288 << 30, 141_100_000_000, 6 << 30
    budget = int(0.9 * total) - weights - act
    n = pages_for_budget(groups, budget, 2, 16, 16384, 256, 16384)[0]
    assert abs(n - budget / per_page) <= 1 and n * 16 > 390_000          # some 400 thousand tokens of context
    # never more than the requests could ever use
    assert pages_for_budget(groups, budget, 2, 16, 2048, 4, 1024)[0] == 4 * 64 + 1
    # a window group takes what its window can hold, the rest share what is left, page for page
    both = [GroupLayout(CacheSpec(8, 128, None), [0, 2], 16), GroupLayout(CacheSpec(8, 128, 64), [1], 16)]
    a, b = pages_for_budget(both, 10 << 20, 2, 16, 128, 4, 4096)
    assert b == ((64 + 128) // 16 + 2) * 4
    assert a == ((10 << 20) - b * both[1].bytes_per_page(2)) // both[0].bytes_per_page(2)
    assert pages_for_budget(groups, -5, 2, 16, 128, 4, 4096) == [0]


def test_replay_pool_holds_max_tokens_at_any_page_size():
    assert pages_for(256, 16) == 16 and pages_for(256, 8) == 32 and pages_for(100, 16) == 7
    assert pages_for(256, 64) == 4 and pages_for(256, 128) == 4      # a request of 64 tokens takes a page of 128
    assert pages_for(256, 24) == 4 * 3                               # 64 tokens end inside a third page of 24


def test_head_sizes_no_kernel_takes_are_refused_when_the_parts_are_built():
    from lmsf_amd.models import DecoderModel
    from lmsf_amd.config import get_architecture
    from lmsf_amd.ops.hip_ops import HipOps
    from lmsf_amd.parts import Runtime

    class Ops:                      # the kernels' own check, without a GPU
        check_head_dim = staticmethod(HipOps.check_head_dim)

    def build(d):
        cfg = LlamaConfig.from_dict(dict(vocab_size=32, hidden_size=24, intermediate_size=16, num_hidden_layers=1,
                                         num_attention_heads=2, num_key_value_heads=1, head_dim=d, rms_norm_eps=1e-5,
                                         max_position_embeddings=32))
        rt = Runtime(ops=Ops(), device=torch.device("cpu"), dtype=torch.float32, max_positions=32)
        return DecoderModel(get_architecture(cfg.architecture).build_spec(cfg), rt)

    build(12)
    build(256)
    for d in (6, 258, 272):
        with pytest.raises(ValueError, match="head size %d is not supported" % d):
            build(d)


def test_float16_runs_as_bfloat16_with_a_warning():
    cfg = LlamaConfig.from_dict(dict(vocab_size=32, hidden_size=16, intermediate_size=16, num_hidden_layers=1,
                                     num_attention_heads=2, num_key_value_heads=1, rms_norm_eps=1e-5,
                                     max_position_embeddings=32, torch_dtype="float16"))
    with pytest.warns(UserWarning, match="runs as bfloat16"):
        assert resolve_dtype(None, cfg) == torch.bfloat16
    assert resolve_dtype("float32", cfg) == torch.float32
