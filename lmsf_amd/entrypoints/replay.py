"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the model,
step function, cache manager and kernels that generation uses. The reference has nothing like
it (its closest is the hand-driven step loop of example/examples/llm_engine_example.rs:65-151).

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
              [--block-size B] [--num-gpu-blocks P] [--random CONFIG.json --seed S]

``--random CONFIG.json`` stands in for ``--model``: the model of that configuration with random weights
made from ``--seed`` (the engine's random-weights mode). ``--block-size`` is the page size in tokens
(default 16); ``--num-gpu-blocks`` sets the number of pages instead of deriving it from ``--max-tokens``.

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries`` gives each request's next tokens and the places among them whose logits are wanted;
all entries of a step run as one batch. ``end`` lists requests that are finished after the step;
their pages go back to the pool. If anything is wanted the step writes ``<out>/<step>.f32``:
little-endian float32 [wanted, vocab], in the order of the entries and of ``want``. After every
step a line ``done <step>`` is printed and flushed.
"""
import argparse
import json
import os
import shutil
import sys
import tempfile
import time

DEFAULT_PAGE_SIZE = 16


def pages_for(max_tokens: int, page_size: int) -> int:
    """Pages that hold ``max_tokens`` tokens of live requests when each request's count is rounded up to a
    multiple of 64: with a page size that divides 64 that is max_tokens / page_size; otherwise every 64
    tokens of a request may end in a page that is partly empty."""
    if 64 % page_size == 0:
        return -(-max_tokens // page_size)
    if page_size % 64 == 0:
        return -(-max_tokens // 64)          # each request rounds up to its own pages: at most one per 64 tokens
    return -(-max_tokens // 64) * -(-64 // page_size)


def _say(msg: str) -> None:
    sys.stderr.write("[trace_run] %s\n" % msg)
    sys.stderr.flush()


def _usable_home() -> None:
    """Libraries may want to write below HOME; with an empty or unwritable one, point it at a temporary folder."""
    home = os.environ.get("HOME", "")
    if not home or not os.path.isdir(home) or not os.access(home, os.W_OK):
        os.environ["HOME"] = tempfile.mkdtemp(prefix="lmsf_home_")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", default=None, help="folder with config.json and model.safetensors")
    ap.add_argument("--random", default=None, metavar="CONFIG.json",
                    help="instead of --model: this configuration with random weights")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights of --random")
    ap.add_argument("--block-size", type=int, default=DEFAULT_PAGE_SIZE, help="tokens a page of the cache holds")
    ap.add_argument("--num-gpu-blocks", type=int, default=None,
                    help="pages of the cache pool (default: what --max-tokens needs)")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time; the cache pool is made for this many")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    if args.max_tokens <= 0:
        ap.error("--max-tokens must be > 0")
    if (args.model is None) == (args.random is None):
        ap.error("give --model DIR or --random CONFIG.json")
    if args.block_size <= 0:
        ap.error("--block-size must be > 0")
    _usable_home()
    os.makedirs(args.out, exist_ok=True)
    t0 = time.time()
    _say("starting (first import of torch can take a minute or two)")
    import torch  # noqa: F401  (the long first import, announced above)

    from lmsf_amd.engine import StepEntry, load_engine_core

    model_dir, load_format = args.model, "auto"
    if args.random is not None:
        model_dir, load_format = tempfile.mkdtemp(prefix="lmsf_random_"), "random"
        shutil.copyfile(args.random, os.path.join(model_dir, "config.json"))
    _say("torch ready after %.0f s; loading kernels and %s" % (time.time() - t0, args.model or args.random))
    num_pages = args.num_gpu_blocks if args.num_gpu_blocks else pages_for(args.max_tokens, args.block_size)
    core = load_engine_core(model_dir, dtype=args.dtype, block_size=args.block_size, num_pages=num_pages,
                            max_num_seqs=64, device=args.device, load_format=load_format, seed=args.seed)
    _say("model %s ready after %.0f s: %s, %d pages of %d tokens" % (
        core.arch.name, time.time() - t0, args.dtype, num_pages, args.block_size))
    executor = core.executor
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        obj = json.loads(line)
        step = obj["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in obj.get("entries", [])]
        logits = executor.step(entries)
        if logits.shape[0] > 0:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            arr.tofile(os.path.join(args.out, "%s.f32" % step))
        for rid in obj.get("end", []):
            executor.release(rid)
        sys.stdout.write("done %s\n" % step)
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
