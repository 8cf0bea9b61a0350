"""The host side of the step function (cache manager, batch building, model assembly) run on the
CPU with torch stand-ins for the kernels, against the plain implementation. The kernels
themselves are tested on the GPU."""

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


def test_padded_batch_sizes_are_few():
    from lmsf_amd.engine.executor import padded_batch
    sizes = sorted({padded_batch(b) for b in range(1, 257)})
    assert sizes == [1, 2, 4, 8] + list(range(16, 257, 8))
    assert all(padded_batch(b) >= b and padded_batch(b) < b + 8 for b in range(1, 257))
    assert padded_batch(5, limit=6) == 6 and padded_batch(300, limit=256) == 300


def test_kinds_of_decode_steps_stay_bounded_and_padding_changes_nothing(tmp_path):
    """Steps of single tokens over a random sequence of batch sizes: the number of kinds the executor keeps
    stays under its limit, all of them write into one logits buffer, and each request's logits are the plain
    implementation's whatever the padding beside it was."""
    import random
    folder, cfg = make_model_folder(tmp_path, "A")
    core = load_engine_core(folder, dtype="float32", block_size=8, num_pages=80, device="cpu", ops=TorchOps(),
                            max_num_seqs=24)
    cfg_dict, w = read_model_folder(folder)
    ex = core.executor
    ex.max_graphs = 3
    assert ex.pad_decode and not ex.use_graphs
    V = cfg_dict["vocab_size"]
    toks = {i: random_tokens(20, V, 50 + i) for i in range(24)}
    ref = {i: plain_llama_forward(cfg_dict, w, t) for i, t in toks.items()}
    ex.step([StepEntry(i, t[:4], []) for i, t in toks.items()])
    at = {i: 4 for i in toks}
    rng = random.Random(1)
    seen = set()
    for _ in range(40):
        ids = rng.sample([i for i in toks if at[i] < 20], k=min(rng.randint(1, 24), sum(a < 20 for a in at.values())))
        out = ex.step([StepEntry(i, toks[i][at[i]:at[i] + 1], [0]) for i in ids])
        seen.update(ex._static)
        assert len(ex._static) <= 3
        for row, i in zip(out, ids):
            assert torch.allclose(row, ref[i][at[i]], atol=2e-5, rtol=1e-5), (i, at[i])
            at[i] += 1
        if all(a >= 20 for a in at.values()):
            break
    assert len(seen) > 3                     # more kinds came by than are kept
    buffers = {sb.device_buffer.data_ptr() for sb in ex._static.values()}
    assert len(buffers) == len(ex._static) and ex._decode_logits.shape[0] == 24
    assert ex.graph_memory_bytes() >= ex._decode_logits.numel() * 4
