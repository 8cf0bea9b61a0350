"""Shared by the tests: the two tiny Llama configurations, model folders, traces."""
import json
import os
import random

import torch

from lmsf_amd.config import LlamaConfig
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

# A wide one: with 17 to 64 tokens in a step its products split K over workgroups and the engine leaves them
# as partial sums for the next kernel, which the narrow configurations never reach.
TINY_W = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=520, hidden_size=1024, intermediate_size=2048,
    num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2, head_dim=128, rms_norm_eps=1e-5,
    rope_theta=10000.0, rope_scaling=None, max_position_embeddings=256, tie_word_embeddings=False,
    attention_bias=True, hidden_act="silu", torch_dtype="float32", bos_token_id=1, eos_token_id=2)

TINY = {"A": (TINY_A, 0, 8), "B": (TINY_B, 1, 16), "C": (TINY_C, 2, 16), "W": (TINY_W, 3, 16)}   # config, seed, block size


def make_model_folder(tmp_path, which, dtype="float32", seed=None, std=0.02):
    """Write config.json + model.safetensors of a tiny configuration; returns (folder, config)."""
    cfg_dict, default_seed, _ = TINY[which]
    cfg = LlamaConfig.from_dict(dict(cfg_dict, torch_dtype=dtype))
    folder = os.path.join(str(tmp_path), "tiny_%s_%s%s" % (which, dtype, "" if std == 0.02 else "_std%g" % std))
    write_random_model(folder, cfg, seed=default_seed if seed is None else seed, dtype=dtype, std=std)
    return folder, cfg


def random_tokens(n, vocab, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


# --------------------------------------------------------------------------- traces
# A trace is a list of steps in trace_run's input form:
#   {"step": i, "entries": [{"id": r, "tokens": [...], "want": [...]}], "end": [r, ...]}
# Every position of every request is wanted, so a replay yields the logits of whole sequences.

def trace_whole(requests):
    """Each request alone and whole, one step each."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def trace_bulk_then_single(requests, tail=32):
    """Most of a request in one step, then its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        cut = max(0, len(toks) - tail)
        parts = ([toks[:cut]] if cut else []) + [[t] for t in toks[cut:]]
        for j, part in enumerate(parts):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": part, "want": list(range(len(part)))}],
                          "end": [rid] if j == len(parts) - 1 else []})
    return steps


def trace_portions(requests, seed=0):
    """Portions of changing size, down to two tokens."""
    rng = random.Random(seed)
    sizes = [17, 5, 64, 3, 2, 31, 2, 16, 15, 1, 33]
    steps = []
    for rid, toks in requests.items():
        at = 0
        while at < len(toks):
            n = min(sizes[rng.randrange(len(sizes))], len(toks) - at)
            last = at + n == len(toks)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at:at + n],
                                                           "want": list(range(n))}], "end": [rid] if last else []})
            at += n
    return steps


def trace_mixed(requests, max_tokens, seed=0, max_live=4, prompt_fraction=0.7):
    """Up to ``max_live`` requests at a time: portions of some beside single tokens of others, requests left
    out of steps now and then, and a pool of ``max_tokens`` so small that pages are used again. A request
    counts with its length rounded up to a multiple of 64."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}     # rid -> [tokens, fed, prompt_len]
    steps = []

    def rounded(n):
        return -(-n // 64) * 64

    while waiting or live:
        while waiting and len(live) < max_live and \
                sum(rounded(len(v[0])) for v in live.values()) + rounded(len(waiting[0][1])) <= max_tokens:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0, max(1, int(len(toks) * prompt_fraction))]
        if not live:
            raise ValueError("a request does not fit max_tokens")
        entries, end = [], []
        rids = list(live)
        chosen = [r for r in rids if rng.random() < 0.8] or [rids[0]]
        for rid in chosen:
            toks, fed, plen = live[rid]
            if fed < plen:
                n = min(rng.choice([2, 3, 7, 16, 24, 40]), plen - fed)
            else:
                n = 1
            entries.append({"id": rid, "tokens": toks[fed:fed + n], "want": list(range(n))})
            live[rid][1] = fed + n
            if fed + n == len(toks):
                end.append(rid)
        for rid in end:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def replay_in_process(executor, steps):
    """Run a trace through a ModelExecutor; returns {request id: float32 logits [len, V]} (CPU)."""
    from lmsf_amd.engine import StepEntry
    got = {}
    for st in steps:
        out = executor.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]]).float().cpu()
        at = 0
        for e in st["entries"]:
            n = len(e["want"])
            got.setdefault(e["id"], []).append(out[at:at + n])
            at += n
        for rid in st["end"]:
            executor.release(rid)
    return {rid: torch.cat(parts) for rid, parts in got.items()}


def replay_with_program(program, model_dir, dtype, steps, out_dir, max_tokens, vocab, timeout=600, extra_args=()):
    """Run a trace through bin/trace_run as a child process; returns {request id: logits [len, V]}."""
    import subprocess

    import numpy as np
    os.makedirs(out_dir, exist_ok=True)
    text = "".join(json.dumps(st) + "\n" for st in steps)
    proc = subprocess.run([program] + (["--model", model_dir] if model_dir else []) + ["--dtype", dtype, "--out", out_dir,
                           "--max-tokens", str(max_tokens)] + list(extra_args), input=text, stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=timeout)
    if proc.returncode != 0:
        raise RuntimeError("trace_run failed (%d):\n%s" % (proc.returncode, proc.stderr[-4000:]))
    done = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert done == ["done %s" % st["step"] for st in steps], proc.stdout[-2000:]
    got = {}
    for st in steps:
        n_want = sum(len(e["want"]) for e in st["entries"])
        path = os.path.join(out_dir, "%s.f32" % st["step"])
        if n_want == 0:
            assert not os.path.exists(path)
            continue
        arr = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
        at = 0
        for e in st["entries"]:
            n = len(e["want"])
            got.setdefault(e["id"], []).append(torch.from_numpy(arr[at:at + n].copy()))
            at += n
    return {rid: torch.cat(parts) for rid, parts in got.items()}
