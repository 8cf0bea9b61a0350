"""Decode and prefill throughput of the engine at Llama-3-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole engine (schedule, batch building, model, sampling) at
batch 8: requests with 512-token random prompts are prefilled (untimed), W decode steps warm up,
then exactly K decode steps are timed between device synchronisations; every step is also timed by
itself with HIP events and the median is reported. The same line carries the prefill of 2,048 tokens,
the decode step's share of the HBM roofline with the machine's measured rates beside the published
peaks, and ``points``: decode at batch 1, 64 and 128, at 8,000 tokens of context, a 512-token prompt,
a mixed step (8 decoding requests beside a 32-token portion of a prompt), continuous batching of
64 requests at Llama-2-7B shape, decode at 32,000 tokens of context, 2,000 short requests with 512 running at a
time, a small model (Llama-3.2-1B sizes) and
the Llama-3.1-70B sizes at all 80 layers (each from an engine of its own, built and dropped in turn). Weights are random (N(0, 0.02), bfloat16, made on the device),
token ids are seeded uniform-random. The reference publishes no numbers, so vs_baseline is null.
"""
import argparse
import json
import os
import random
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

TUNE_PRODUCTS = True      # --no-tune: the BLAS library's own choice of algorithm for the prefill steps' products

LLAMA3_8B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=4096,
    intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
    rms_norm_eps=1e-5, rope_theta=500000.0, rope_scaling=None, max_position_embeddings=8192,
    tie_word_embeddings=False, attention_bias=False, hidden_act="silu", torch_dtype="bfloat16",
    bos_token_id=128000, eos_token_id=128001)


def make_engine(cfg, args, max_num_seqs, dtype, prefill_chunk_size=None):
    from lmsf_amd.engine import EngineArgs, LLMEngine
    folder = tempfile.mkdtemp(prefix="lmsf_bench_")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    return LLMEngine(EngineArgs(model=folder, dtype=dtype, block_size=getattr(args, "block_size", 16), load_format="random", seed=0,
                                max_num_seqs=max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens,
                                gpu_memory_utilization=args.gpu_memory_utilization,
                                prefill_chunk_size=prefill_chunk_size))


def weight_bytes(engine):
    """Bytes of every weight a decode step reads once: all matrices and norm weights, the LM head, not
    the embedding table (one row per token)."""
    seen, total = set(), 0
    model = engine.core.model
    head = {t.data_ptr() for t in model.head.tensors()}
    gathered = {t.data_ptr() for t in model.embedding.tensors()} - head     # (tied: the head reads the table whole)
    for p in model.parts():
        for t in p.tensors():
            if t.data_ptr() in seen or t.data_ptr() in gathered:
                continue
            seen.add(t.data_ptr())
            total += t.numel() * t.element_size()
    return total


def decode_run(engine, batch, prompt_len, steps, warmup, seed):
    """Prefill ``batch`` prompts, warm up, time ``steps`` decode steps. Returns (seconds, mean context)."""
    import torch
    from lmsf_amd.sampling import SamplingParams
    rng = random.Random(seed)
    V = engine.core.config.vocab_size
    ids = []
    # requests whose prompts are done first decode while the others are still being prefilled: room for that
    slack = batch * prompt_len // 1024 + 16
    for i in range(batch):
        rid = "b%d_%d" % (batch, i)
        engine.add_request(rid, [rng.randrange(V) for _ in range(prompt_len)],
                           SamplingParams(temperature=0.0, max_tokens=steps + warmup + slack, ignore_eos=True))
        ids.append(rid)
    while any(s.remaining > 1 for s in list(engine.scheduler.running) + list(engine.scheduler.waiting)) \
            or engine.scheduler.waiting:
        engine.step()
    for _ in range(warmup):
        engine.step()
    ctx0 = sum(s.length for s in engine.scheduler.running) / batch
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for a, b in events:
        a.record()
        outs = engine.step()
        b.record()
        assert len(outs) == batch
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for rid in ids:
        engine.abort_request(rid)
    per_step = sorted(a.elapsed_time(b) for a, b in events)
    decode_run.median_ms = per_step[len(per_step) // 2]
    return dt, ctx0 + steps / 2.0


def prefill_run(engine, n_tokens, reps, seed):
    """Median seconds of a prefill of ``n_tokens`` tokens of one request (one step, logits of the last token)."""
    import torch
    from lmsf_amd.engine import StepEntry
    rng = random.Random(seed)
    V = engine.core.config.vocab_size
    times = []
    if TUNE_PRODUCTS:
        # the library's candidates for this step's products race first, as the engine does at load for its full
        # step with EngineArgs.tune_products
        engine.core.executor.tune_products([n_tokens])
    for r in range(reps + 1):
        toks = [rng.randrange(V) for _ in range(n_tokens)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.core.executor.step([StepEntry("prefill", toks, [n_tokens - 1])])
        torch.cuda.synchronize()
        if r > 0:
            times.append(time.perf_counter() - t0)
        engine.core.executor.release("prefill")
    times.sort()
    return times[len(times) // 2]


def mixed_step_run(engine, n_decoding, context, portion, reps, seed):
    """A step of ``n_decoding`` single tokens (requests with ``context`` tokens behind them) beside a
    ``portion``-token piece of a prompt, through the step function: (median milliseconds from call to
    synchronised result, median milliseconds on the GPU by events)."""
    import torch
    from lmsf_amd.engine import StepEntry
    rng = random.Random(seed)
    V = engine.core.config.vocab_size
    ex = engine.core.executor
    ids = ["m%d" % i for i in range(n_decoding)]
    for rid in ids:
        ex.step([StepEntry(rid, [rng.randrange(V) for _ in range(context)], [])])
    ex.step([StepEntry("mp", [rng.randrange(V) for _ in range(context)], [])])

    def entries():
        e = [StepEntry(rid, [rng.randrange(V)], [0]) for rid in ids]
        e.append(StepEntry("mp", [rng.randrange(V) for _ in range(portion)], [portion - 1]))
        return e
    wall, gpu = [], []
    for r in range(reps + 2):
        e = entries()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        a.record()
        ex.step(e)
        b.record()
        torch.cuda.synchronize()
        if r >= 2:
            wall.append((time.perf_counter() - t0) * 1e3)
            gpu.append(a.elapsed_time(b))
    for rid in ids + ["mp"]:
        ex.release(rid)
    wall.sort(), gpu.sort()
    return wall[len(wall) // 2], gpu[len(gpu) // 2]


LLAMA2_7B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=32000, hidden_size=4096,
    intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=32, head_dim=128,
    rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, max_position_embeddings=4096,
    tie_word_embeddings=False, attention_bias=False, hidden_act="silu", torch_dtype="bfloat16",
    bos_token_id=1, eos_token_id=2)


LLAMA31_70B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=8192,
    intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
    rms_norm_eps=1e-5, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=16384, tie_word_embeddings=False, attention_bias=False, hidden_act="silu",
    torch_dtype="bfloat16", bos_token_id=128000, eos_token_id=128001)

# a small model of the same architecture: head size 64, tied embeddings, few and narrow layers (launches count)
LLAMA32_1B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=2048,
    intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
    rms_norm_eps=1e-5, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    max_position_embeddings=16384, tie_word_embeddings=True, attention_bias=False, hidden_act="silu",
    torch_dtype="bfloat16", bos_token_id=128000, eos_token_id=128001)

SHAPES = {"llama3-8b": ("Llama-3-8B", LLAMA3_8B), "llama2-7b": ("Llama-2-7B", LLAMA2_7B),
          "llama3.1-70b": ("Llama-3.1-70B", LLAMA31_70B), "llama3.2-1b": ("Llama-3.2-1B", LLAMA32_1B)}


def serve_run(args, emit=True):
    """Continuous batching at Llama-2-7B shape: 64 requests arrive at once, prompts of 128 to 2,048 random
    tokens, 128 generated tokens each, prompts cut into portions that run beside the decoding requests."""
    import torch
    from lmsf_amd.sampling import SamplingParams
    cfg = dict(LLAMA2_7B)
    if args.layers and emit:
        cfg["num_hidden_layers"] = args.layers
    engine = make_engine(cfg, args, max_num_seqs=64, dtype=args.dtype, prefill_chunk_size=args.prefill_chunk_size)
    rng = random.Random(7)
    V = cfg["vocab_size"]

    def load(n_req, n_out):
        prompts = [[rng.randrange(V) for _ in range(rng.randint(128, 2048))] for _ in range(n_req)]
        for i, p in enumerate(prompts):
            engine.add_request("s%d_%d" % (n_req, i), p, SamplingParams(temperature=0.0, max_tokens=n_out, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = 0
        while engine.has_unfinished_requests():
            engine.step()
            steps += 1
        torch.cuda.synchronize()
        return time.perf_counter() - t0, steps, sum(len(p) for p in prompts)

    load(8, 8)                                   # warm-up: kernels, graphs of the small batch sizes
    dt, steps, prompt_tokens = load(64, 128)
    out_tokens = 64 * 128
    line = {
        "metric": "continuous batching, generated tok/s (Llama-2-7B bf16, 64 requests)", "value": round(out_tokens / dt, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 0, "ms_per_step": round(dt / steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": "Llama-2-7B shape, random weights", "global_batch": 64, "seq_len": 2048,
                   "parallelism": "single GPU", "layers": cfg["num_hidden_layers"], "layers_of_model": 32,
                   "requests": 64, "prompt_tokens": prompt_tokens, "generated_tokens": out_tokens,
                   "prefill_chunk_size": args.prefill_chunk_size, "max_num_batched_tokens": args.max_num_batched_tokens,
                   "total_tok_per_s": round((prompt_tokens + out_tokens) / dt, 1), "seconds": round(dt, 3),
                   "preemptions": engine.stats["preemptions"]},
    }
    if emit:
        print(json.dumps(line))
    return line


def products_run(args):
    """The four matrix products of a layer at the headline shape, for some numbers of rows: the BLAS library's
    (through torch) against this package's choice (``HipOps.linear`` / ``linear_gated``). Microseconds by HIP
    events around a HIP graph of eight calls (no host time between the kernels), the weight read from memory
    every time. One JSON line per product and number of rows."""
    import torch
    from lmsf_amd.ops import get_ops
    ops = get_ops()
    cfg = SHAPES[args.shape][1]
    H, I = cfg["hidden_size"], cfg["intermediate_size"]
    d, nh, nkv = cfg["head_dim"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    shapes = {"qkv": ((nh + 2 * nkv) * d, H, False), "o": (H, nh * d, False), "gate_up": (2 * I, H, True),
              "down": (H, I, False)}
    g = torch.Generator(device="cuda:0").manual_seed(1)

    def timed(f, reps=8):
        """Microseconds a call: ``reps`` calls recorded into a HIP graph once (no host time between the kernels),
        replayed six times between events; the median."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                f()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(reps):
                f()
        times = []
        for _ in range(6):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            b.synchronize()
            times.append(a.elapsed_time(b) / reps)
        del graph
        return sorted(times)[len(times) // 2] * 1e3
    for name, (N, K, gated) in shapes.items():
        # rows as far apart as the engine lays a weight's rows out
        pad = ops.weight_row_pad(K, torch.bfloat16)

        def laid_out(t):
            buf = torch.empty(N, K + pad, dtype=torch.bfloat16, device="cuda:0")
            buf[:, :K].copy_(t)
            return buf[:, :K]
        W = laid_out(torch.randn(N, K, device="cuda:0", generator=g) * 0.02)
        # as in a model, every call streams its weight from memory: the copies in turn are larger together than
        # the 256 MB of the memory-side cache
        copies = [W] + [laid_out(W) for _ in range(int(1.5e9 // (N * K * 2)))]
        turn = [0]

        def weight():
            turn[0] = (turn[0] + 1) % len(copies)
            return copies[turn[0]]
        for M in [int(m) for m in args.rows.split(",")]:
            x = torch.randn(M, K, device="cuda:0", generator=g).to(torch.bfloat16)
            if gated:
                lib = lambda w: ops.gated_act(torch.nn.functional.linear(x, w), "silu")    # noqa: E731
                own = lambda w: ops.linear_gated(x, w, None, "silu")                          # noqa: E731
            else:
                lib = lambda w: torch.nn.functional.linear(x, w)                              # noqa: E731
                own = lambda w: ops.linear(x, w)                                              # noqa: E731
            a, b = own(W).float(), lib(W).float()
            err = (a - b).abs().max().item() / b.abs().max().item()
            t_lib, t_own = timed(lambda: lib(weight())), timed(lambda: own(weight()))
            flops = 2.0 * M * N * K
            print(json.dumps({"product": name, "rows": M, "N": N, "K": K, "library_us": round(t_lib, 1),
                              "library_PFLOPs": round(flops / t_lib / 1e9, 3), "engine_us": round(t_own, 1),
                              "engine_PFLOPs": round(flops / t_own / 1e9, 3), "max_diff_of_largest": err}))
            del a, b


def further_shape_points(args, points, peak):
    """Points at other sizes than the headline's, each from an engine of its own that is built and dropped in
    turn: decode at 32,000 tokens of context (batch 8, the headline shape with room for such contexts), a small
    model (Llama-3.2-1B sizes: launches count) at batch 1 and 64, and the Llama-3.1-70B sizes at all 80 layers
    (141 GB of weights) at batch 1 and 8 with a 2,048-token prefill. Every rate comes with its share of the roofline."""
    import gc
    import torch

    def with_engine(cfg, max_seqs, fn, utilization=None):
        a = argparse.Namespace(**vars(args))
        if utilization:
            a.gpu_memory_utilization = utilization
        try:
            engine = make_engine(cfg, a, max_num_seqs=max_seqs, dtype=args.dtype)
        except Exception as e:  # noqa: BLE001 - a point that cannot be measured is named, the line is still printed
            return "%s: %s" % (type(e).__name__, str(e)[:160])
        try:
            fn(engine)
        finally:
            del engine
            gc.collect()
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
        return None

    es = 2 if args.dtype == "bfloat16" else 4

    def decode_point(engine, cfg, name, batch, prompt_len, steps, warmup, seed):
        kv = 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * cfg["num_hidden_layers"] * es
        d, ctx = decode_run(engine, batch, prompt_len, steps, warmup, seed=seed)
        points[name] = round(batch * steps / d, 1)
        points[name + "_hbm_frac"] = round((weight_bytes(engine) + batch * ctx * kv) / (d / steps) / HBM_BYTES_PER_S, 4)

    long_cfg = dict(LLAMA3_8B, max_position_embeddings=32768 + 64)
    err = with_engine(long_cfg, 8, lambda e: decode_point(e, long_cfg, "decode_b8_ctx32000", 8, 32000, 16, 4, 71))
    if err:
        points["decode_b8_ctx32000_error"] = err

    def short_requests(e):
        """Thousands of short requests at once at the headline shape: 2,000 requests of 32 to 96 prompt tokens and
        16 to 32 generated, 512 running at a time; every step holds the decoding requests beside the prompts of
        those just admitted, about 1,500 tokens."""
        from lmsf_amd.sampling import SamplingParams
        rng = random.Random(5)
        V = LLAMA3_8B["vocab_size"]

        def load(n_req, tag):
            for i in range(n_req):
                prompt = [rng.randrange(V) for _ in range(rng.randint(32, 96))]
                e.add_request("%s%d" % (tag, i), prompt,
                              SamplingParams(temperature=0.0, max_tokens=rng.randint(16, 32), ignore_eos=True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            steps = generated = 0
            while e.has_unfinished_requests():
                generated += len(e.step())
                steps += 1
            torch.cuda.synchronize()
            return time.perf_counter() - t0, steps, generated
        load(16, "w")
        dt, steps, generated = load(2000, "q")
        points["short_requests_tok_s"] = round(generated / dt, 1)
        points["short_requests_running"] = 512
        points["short_requests_ms_per_step"] = round(dt / steps * 1e3, 3)
    err = with_engine(dict(LLAMA3_8B), 512, short_requests)
    if err:
        points["short_requests_error"] = err

    small = dict(LLAMA32_1B)

    def small_points(e):
        decode_point(e, small, "llama1b_decode_b1", 1, 512, 32, 8, 72)
        decode_point(e, small, "llama1b_decode_b64", 64, 512, 32, 8, 73)
    err = with_engine(small, 64, small_points)
    if err:
        points["llama1b_error"] = err

    big = dict(LLAMA31_70B)

    def big_points(e):
        points["llama70b_layers"] = big["num_hidden_layers"]
        decode_point(e, big, "llama70b_decode_b1", 1, 512, 12, 3, 74)
        decode_point(e, big, "llama70b_decode_b8", 8, 512, 12, 3, 75)
        t = prefill_run(e, 2048, reps=3, seed=76)
        points["llama70b_prefill_2048_tok_s"] = round(2048 / t, 1)
        points["llama70b_prefill_2048_frac"] = round(prefill_flops(big, 2048) / t / peak, 4)
    err = with_engine(big, 8, big_points, utilization=0.9)
    if err:
        points["llama70b_error"] = err


def prefill_flops(cfg, T):
    """Multiply-adds times two of a causal prefill of T tokens: the linear layers on every token, the
    attention scores and values over the causal half, the LM head on one row."""
    H, I, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["num_hidden_layers"]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    per_token = L * ((nh + 2 * nkv) * d * H + nh * d * H + 3 * I * H)
    attn = L * nh * d * 2 * (T * (T + 1) // 2)
    return 2.0 * (per_token * T + attn + cfg["vocab_size"] * H)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--max-num-batched-tokens", type=int, default=8192)
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.85)
    ap.add_argument("--skip-points", action="store_true", help="leave out the batch 1 and batch 64 runs")
    ap.add_argument("--workload", default="decode", choices=["decode", "serve", "products"],
                    help="decode: the default line (Llama-3-8B shape); serve: continuous batching of 64 requests at "
                         "Llama-2-7B shape, a line of its own; products: a layer's matrix products alone, the "
                         "library's against the engine's choice, at --rows")
    ap.add_argument("--rows", default="17,64,100,128,129,192,256,512,2048", help="products: numbers of rows")
    ap.add_argument("--prefill-chunk-size", type=int, default=1024, help="serve: longest portion of a prompt in a step")
    ap.add_argument("--shape", default="llama3-8b", choices=sorted(SHAPES),
                    help="decode: the model whose layer sizes are measured (default: the headline configuration)")
    ap.add_argument("--tunable", action="append", default=[], metavar="NAME=INT",
                    help="set an attribute of ops.HipOps (a number of rows at which kernels change, a variant) first")
    ap.add_argument("--points", default="1,64,128", help="decode: further batch sizes, comma separated")
    ap.add_argument("--block-size", type=int, default=16, help="tokens a page of the cache")
    ap.add_argument("--no-tune", action="store_true",
                    help="leave the BLAS library's choice of algorithm as it is (default: its candidates race for the "
                         "shapes of the prefill steps, as EngineArgs.tune_products does at load)")
    ap.add_argument("--max-context", type=int, default=None,
                    help="decode: positions the model allows, for --prompt-len beyond the shape's own "
                         "(--batch 1 --prompt-len 120000 --max-context 131072 --skip-points)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus)
        sys.exit(2)

    global TUNE_PRODUCTS
    TUNE_PRODUCTS = not args.no_tune
    if args.tunable:
        from lmsf_amd.ops import get_ops
        ops = get_ops()
        for item in args.tunable:
            name, _, value = item.partition("=")
            if not hasattr(ops, name) or not isinstance(getattr(ops, name), int):
                raise SystemExit("bench.py: HipOps has no integer attribute %r" % name)
            setattr(ops, name, int(value))
    if args.workload == "serve":
        serve_run(args)
        return
    if args.workload == "products":
        products_run(args)
        return
    import torch
    shape_name, shape_cfg = SHAPES[args.shape]
    cfg = dict(shape_cfg)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    if args.max_context:
        cfg["max_position_embeddings"] = args.max_context
    point_batches = [] if args.skip_points else [int(x) for x in args.points.split(",") if x]
    max_seqs = max([64, args.batch] + point_batches)
    engine = make_engine(cfg, args, max_num_seqs=max_seqs, dtype=args.dtype)
    wbytes = weight_bytes(engine)
    cache_pages = engine.core.storage.groups[0].num_pages if engine.core.storage.groups else 0
    kv_per_token = 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * cfg["num_hidden_layers"] * \
        (2 if args.dtype == "bfloat16" else 4)

    measured = engine.core.rt.ops.measure()

    dt, mean_ctx = decode_run(engine, args.batch, args.prompt_len, args.steps, args.warmup, seed=1)
    ms_per_step = dt / args.steps * 1e3
    median_ms = decode_run.median_ms
    value = args.batch * args.steps / dt
    step_bytes = wbytes + args.batch * mean_ctx * kv_per_token
    achieved = step_bytes / (dt / args.steps) / 1e9

    points = {"decode_b%d_median_ms" % args.batch: round(median_ms, 4)}
    if not args.skip_points:
        for b in point_batches:
            k = max(16, args.steps // 2)
            d, ctx_b = decode_run(engine, b, args.prompt_len, k, args.warmup, seed=2 + b)
            points["decode_b%d" % b] = round(b * k / d, 1)
            points["decode_b%d_hbm_frac" % b] = round((wbytes + b * ctx_b * kv_per_token) / (d / k) / HBM_BYTES_PER_S, 4)
        long_ctx = min(8000, cfg["max_position_embeddings"] - 64)
        for b in (1, 8):
            d, ctx_b = decode_run(engine, b, long_ctx, 24, 4, seed=40 + b)
            points["decode_b%d_ctx%d" % (b, long_ctx)] = round(b * 24 / d, 1)
            points["decode_b%d_ctx%d_hbm_frac" % (b, long_ctx)] = round(
                (wbytes + b * ctx_b * kv_per_token) / (d / 24) / HBM_BYTES_PER_S, 4)
        wall_ms, gpu_ms = mixed_step_run(engine, 8, args.prompt_len, 32, reps=9, seed=5)
        points["mixed_step_ms"] = round(wall_ms, 3)
        points["mixed_step_gpu_ms"] = round(gpu_ms, 3)

    pt = prefill_run(engine, args.prefill_tokens, reps=5, seed=3)
    pflops = prefill_flops(cfg, args.prefill_tokens)
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    if not args.skip_points:
        p512 = prefill_run(engine, 512, reps=5, seed=4)
        points["prefill_512_tok_s"] = round(512 / p512, 1)
        points["prefill_512_frac"] = round(prefill_flops(cfg, 512) / p512 / peak, 4)
        long_prompt = min(8192, args.max_num_batched_tokens, cfg["max_position_embeddings"])
        if long_prompt > args.prefill_tokens:
            pl = prefill_run(engine, long_prompt, reps=3, seed=6)
            points["prefill_%d_tok_s" % long_prompt] = round(long_prompt / pl, 1)
            points["prefill_%d_frac" % long_prompt] = round(prefill_flops(cfg, long_prompt) / pl / peak, 4)
        if args.shape == "llama3-8b" and args.dtype == "bfloat16":
            # continuous batching at Llama-2-7B shape needs the memory: the first engine goes
            del engine
            import gc
            gc.collect()
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            held = torch.cuda.memory_allocated()
            if held > (2 << 30):
                print("bench: %.1f GB of the first engine are still held when the serving point starts"
                      % (held / 2 ** 30), file=sys.stderr)
            serve = serve_run(args, emit=False)
            points["serve_tok_s"] = serve["value"]
            points["serve_total_tok_s"] = serve["config"]["total_tok_per_s"]
            points["serve_ms_per_step"] = serve["ms_per_step"]
            points["serve_preemptions"] = serve["config"]["preemptions"]
            further_shape_points(args, points, peak)

    line = {
        "metric": "decode tok/s at batch %d (%s %s)" % (args.batch, shape_name, "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": "%s shape, random weights" % shape_name, "global_batch": args.batch, "seq_len": args.prompt_len,
            "parallelism": "single GPU", "layers": cfg["num_hidden_layers"], "layers_of_model": full_layers,
            "hidden_size": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
            "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate_size": cfg["intermediate_size"], "vocab_size": cfg["vocab_size"],
            "max_context": cfg["max_position_embeddings"], "block_size": args.block_size, "prompt_len": args.prompt_len,
            "mean_decode_context": round(mean_ctx, 1), "prefill_tokens": args.prefill_tokens,
            "cache_pages": cache_pages, "gpu_memory_utilization": args.gpu_memory_utilization,
        },
        "prefill": {"value": round(args.prefill_tokens / pt, 1), "tokens": args.prefill_tokens,
                    "ms": round(pt * 1e3, 3), "frac": round(pflops / pt / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": round(achieved / (HBM_BYTES_PER_S / 1e9), 4),
                     "measured_read_GBps": round(measured["read_GBps"], 1),
                     "measured_copy_GBps": round(measured["copy_GBps"], 1),
                     "measured_mfma_bf16_TFLOPs": round(measured["mfma_bf16_TFLOPs"], 1),
                     "nominal_mfma_bf16_TFLOPs": PEAK_FLOPS["bf16"] / 1e12},
        "points": points,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
