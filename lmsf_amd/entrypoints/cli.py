"""Command line in the manner of the reference's llm_engine_example
(example/examples/llm_engine_example.rs:9-151): engine options with the reference's names, one
request (or several) with the example's sampling defaults (temperature 0.8, top_k 5,
presence_penalty 0.2, max_tokens 16), output printed as it is produced, then the time it cost.
A prompt is text (``--prompt``, the example's own is "To be or not to be,") if the model folder has a
tokenizer.json, or token ids.

    lmsf_generate --model DIR --gpu-memory-utilization 0.95 --block-size 8 --max-model-len 1024 \\
        --prompt "To be or not to be,"
    lmsf_generate --model DIR --prompt-ids 1,15043,3186
"""
import argparse
import random
import sys
import time
from typing import List


def _parse_ids(text: str) -> List[int]:
    return [int(x) for x in text.replace(",", " ").split()]


def build_parser() -> argparse.ArgumentParser:
    from lmsf_amd.engine.args import EngineArgs
    ap = argparse.ArgumentParser(prog="lmsf_generate", description=__doc__.split("\n\n")[0])
    EngineArgs.add_cli_args(ap)
    g = ap.add_argument_group("requests")
    g.add_argument("--prompt", action="append", default=[], help="a prompt as text (repeatable; needs tokenizer.json)")
    g.add_argument("--prompt-ids", action="append", default=[], help="a prompt as comma-separated token ids (repeatable)")
    g.add_argument("--prompt-file", default=None, help="file with one prompt per line, token ids separated by blanks or commas")
    g.add_argument("--random-prompts", type=int, default=0, help="number of random prompts to add")
    g.add_argument("--random-prompt-len", type=int, default=16)
    s = ap.add_argument_group("sampling")
    s.add_argument("--temperature", type=float, default=0.8)
    s.add_argument("--top-k", type=int, default=5)
    s.add_argument("--top-p", type=float, default=1.0)
    s.add_argument("--min-p", type=float, default=0.0)
    s.add_argument("--presence-penalty", type=float, default=0.2)
    s.add_argument("--frequency-penalty", type=float, default=0.0)
    s.add_argument("--repetition-penalty", type=float, default=1.0)
    s.add_argument("--max-tokens", type=int, default=16)
    s.add_argument("--ignore-eos", action="store_true")
    s.add_argument("--stop", action="append", default=[], help="a string that ends the output (repeatable)")
    s.add_argument("--include-stop-str-in-output", action="store_true")
    s.add_argument("--sampling-seed", type=int, default=None, help="seed of every request's draws (default: from --seed)")
    return ap


def main(argv=None) -> int:
    ap = build_parser()
    ns = ap.parse_args(argv)
    from lmsf_amd.engine import EngineArgs, LLMEngine
    from lmsf_amd.sampling import SamplingParams

    prompts = list(ns.prompt) + [_parse_ids(p) for p in ns.prompt_ids]
    if ns.prompt_file:
        with open(ns.prompt_file) as f:
            prompts += [_parse_ids(line) for line in f if line.strip()]
    args = EngineArgs.from_cli_args(ns)
    t0 = time.time()
    engine = LLMEngine(args)
    sys.stderr.write("engine ready in %.1f s: %s, %s, context %d\n" % (
        time.time() - t0, engine.core.arch.name, str(engine.core.rt.dtype).replace("torch.", ""),
        engine.core.max_model_len))
    if ns.random_prompts:
        rng = random.Random(ns.seed)
        V = engine.core.config.vocab_size
        prompts += [[rng.randrange(V) for _ in range(ns.random_prompt_len)] for _ in range(ns.random_prompts)]
    if not prompts:
        ap.error("no prompt given (--prompt, --prompt-ids, --prompt-file or --random-prompts)")
    for i, p in enumerate(prompts):
        engine.add_request(i, p, SamplingParams(
            temperature=ns.temperature, top_k=ns.top_k, top_p=ns.top_p, min_p=ns.min_p,
            presence_penalty=ns.presence_penalty, frequency_penalty=ns.frequency_penalty,
            repetition_penalty=ns.repetition_penalty, max_tokens=ns.max_tokens, ignore_eos=ns.ignore_eos,
            stop=list(ns.stop), include_stop_str_in_output=ns.include_stop_str_in_output, seed=ns.sampling_seed))
    start = time.time()
    n_tokens = 0
    finals = {}
    while engine.has_unfinished_requests():
        for out in engine.step():
            for c in out.outputs:
                if c.latest_token is not None:
                    n_tokens += 1
                    if len(prompts) == 1:
                        sys.stdout.write(c.latest_text if engine.tokenizer is not None else "%d " % c.latest_token)
                        sys.stdout.flush()
            if out.finished:
                finals[out.request_id] = out
    if len(prompts) == 1:
        sys.stdout.write("\n")
    else:
        for rid in sorted(finals):
            o = finals[rid].outputs[0]
            shown = o.text if engine.tokenizer is not None else " ".join(str(t) for t in o.token_ids)
            print("[%s] %s (%s)" % (rid, shown, o.finish_reason))
    cost = time.time() - start
    print("cost %.3f s to gen %d tokens (%.1f tokens/s, %d steps, %d preemptions)" % (
        cost, n_tokens, n_tokens / max(cost, 1e-9), engine.stats["steps"], engine.stats["preemptions"]))
    return 0


if __name__ == "__main__":
    sys.exit(main())
