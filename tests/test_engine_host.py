"""The host side of the step function (cache manager, batch building, model assembly) run on the
CPU with torch stand-ins for the kernels, against the plain implementation. The kernels
themselves are tested on the GPU."""
import os

import pytest
import torch

from helpers import TINY, make_model_folder, random_tokens
from plain_llama import plain_llama_forward, read_model_folder
from torch_ops import TorchOps

from lmsf_amd.cache import OutOfPages
from lmsf_amd.engine import StepEntry, load_engine_core


def build(tmp_path, which, num_pages, max_model_len=None):
    folder, cfg = make_model_folder(tmp_path, which)
    core = load_engine_core(folder, dtype="float32", block_size=TINY[which][2], num_pages=num_pages,
                            max_model_len=max_model_len, device="cpu", ops=TorchOps(), max_num_seqs=8)
    cfg_dict, weights = read_model_folder(folder)
    return core, cfg_dict, weights


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_whole_prompt_matches_plain(tmp_path, which):
    core, cfg, w = build(tmp_path, which, num_pages=16)
    toks = random_tokens(37, cfg["vocab_size"], 3)
    logits = core.executor.step([StepEntry("r", toks, list(range(len(toks))))])
    ref = plain_llama_forward(cfg, w, toks)
    assert torch.allclose(logits, ref, atol=2e-5, rtol=1e-5), (logits - ref).abs().max()


@pytest.mark.parametrize("which", ["A", "B"])
def test_portions_and_decode_match_whole(tmp_path, which):
    core, cfg, w = build(tmp_path, which, num_pages=16)
    toks = random_tokens(50, cfg["vocab_size"], 4)
    ref = plain_llama_forward(cfg, w, toks)
    got = []
    cuts = [17, 5, 2, 9, 3]
    at = 0
    for c in cuts:
        got.append(core.executor.step([StepEntry("r", toks[at:at + c], list(range(c)))]))
        at += c
    while at < len(toks):
        got.append(core.executor.step([StepEntry("r", toks[at:at + 1], [0])]))
        at += 1
    got = torch.cat(got)
    assert torch.allclose(got, ref, atol=2e-5, rtol=1e-5), (got - ref).abs().max()


def test_mixed_batch_with_page_reuse(tmp_path):
    which = "B"
    core, cfg, w = build(tmp_path, which, num_pages=12)    # 192 tokens of room
    V = cfg["vocab_size"]
    a, b, c = random_tokens(90, V, 5), random_tokens(70, V, 6), random_tokens(80, V, 7)
    ref = {k: plain_llama_forward(cfg, w, t) for k, t in (("a", a), ("b", b), ("c", c))}
    ex = core.executor
    got = {"a": [], "b": [], "c": []}

    def run(entries):
        out = ex.step([StepEntry(k, t, want) for k, t, want in entries])
        at = 0
        for k, t, want in entries:
            got[k].append(out[at:at + len(want)])
            at += len(want)

    run([("a", a[:60], list(range(60))), ("b", b[:20], list(range(20)))])
    run([("a", a[60:61], [0]), ("b", b[20:70], list(range(50)))])
    for i in range(61, 90):
        run([("a", a[i:i + 1], [0])])
    ex.release("b")
    ex.release("a")
    core.storage.manager.check_invariants()
    run([("c", c[:33], list(range(33)))])          # reuses pages a and b gave back
    run([("c", c[33:], list(range(len(c) - 33)))])
    for k in ("a", "b", "c"):
        g = torch.cat(got[k])
        assert torch.allclose(g, ref[k], atol=2e-5, rtol=1e-5), (k, (g - ref[k]).abs().max())
    ex.release("c")
    core.storage.manager.check_invariants()
    assert core.storage.manager.num_free_pages(0) == 12


def test_out_of_pages_takes_nothing(tmp_path):
    core, cfg, _ = build(tmp_path, "A", num_pages=4)       # 32 tokens
    V = cfg["vocab_size"]
    ex = core.executor
    ex.step([StepEntry("x", random_tokens(20, V, 1), [19])])
    with pytest.raises(OutOfPages):
        ex.step([StepEntry("x", random_tokens(4, V, 2), [3]), StepEntry("y", random_tokens(16, V, 3), [15])])
    mgr = core.storage.manager
    mgr.check_invariants()
    assert mgr.num_tokens("x") == 20 and not mgr.has_request("y")
    assert mgr.num_free_pages(0) == 1
