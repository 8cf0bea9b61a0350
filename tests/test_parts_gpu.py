"""The parts a model is put together from, each alone against the plain implementation; models put
together differently from the same parts (a layer twice, a layer reading another layer's cache, a
window); and toy parts defined here (a mixer with state of its own, a feed-forward with routing,
another position encoding) registered, built and stepped without touching the package."""

import pytest
import torch

import plain_llama as P
from helpers import (TINY, TINY_B, make_model_folder, random_tokens, replay_in_process, trace_bulk_then_single,
                     trace_mixed, trace_portions, trace_whole)

from lmsf_amd.config import LlamaConfig, register_architecture, unregister_architecture
from lmsf_amd.engine import GroupView, StepContext, StepEntry, load_engine_core
from lmsf_amd.models.llama import build_llama_spec
from lmsf_amd.parts import (CacheBinding, FeedForward, LayerSpec, Mixer, ModelSpec, PartSpec, PositionEncoding,
                            Runtime, ScheduleEntry, StateSpec, TensorDecl, build_part, register_part, unregister_part)
from lmsf_amd.weights import write_random_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)


def close(got, want, dtype):
    """float32: element by element. bfloat16: a part rounds its intermediate results to 8 bits of mantissa, so
    a sum over a row carries an error in proportion to the row's size, not to the element's: the bound is
    relative to the largest value."""
    got, want = got.float().cpu(), want.float()
    if dtype == torch.float32:
        return torch.allclose(got, want, atol=3e-5, rtol=3e-5)
    return (got - want).abs().max().item() <= 1.5e-2 * max(1.0, want.abs().max().item())


def runtime(dtype, max_positions=256):
    from lmsf_amd.ops import get_ops
    return Runtime(ops=get_ops(), device=torch.device(DEV), dtype=dtype, max_positions=max_positions)


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def give(part, tensors, dtype):
    """Load a part (and its children) from a dict of float32 CPU tensors, rounded to ``dtype`` as a checkpoint
    in that dtype would be."""
    for p in part.walk():
        p.load_weights(lambda name: tensors[name].to(dtype).to(DEV))


def rounded(t, dtype):
    return t.to(dtype).float()


def whole_prompt_context(T, page_size, first_pos=0):
    """The batch description of one request's T tokens standing at first_pos .. first_pos + T - 1, pages in order."""
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    n_pages = -(-(first_pos + T) // page_size)
    return StepContext(
        n_tokens=T, n_segments=1, token_ids=i32([0] * T), positions=i32(list(range(first_pos, first_pos + T))),
        seg_of_token=i32([0] * T), seg_starts=i32([0, T]), seg_first_pos=i32([first_pos]), state_slots=i32([0]),
        logit_rows=i32(list(range(T))), n_logit_rows=T,
        groups=[GroupView(slots=i32(list(range(first_pos, first_pos + T))), block_tables=i32([list(range(n_pages))]),
                          page_size=page_size)],
        host_seg_starts=[0, T], host_seg_lens=[T], host_seg_first_pos=[first_pos], host_state_slots=[0],
        request_ids=["r"], max_seg_len=T, max_context=first_pos + T, all_single=T == 1), n_pages


# --------------------------------------------------------------------------- each part alone

@pytest.mark.parametrize("dtype", DTYPES)
def test_rms_norm_part(dtype):
    rt = runtime(dtype)
    H, eps = 80, 3e-6
    norm = build_part("norm", PartSpec("rms_norm", {"size": H, "eps": eps}), "n", rt)
    assert norm.checkpoint_tensors() == {"n.weight": TensorDecl((H,), init="ones", keeps_float32=True)}
    w = rnd(H, seed=1) + 1.0
    give(norm, {"n.weight": w}, dtype)
    x = rnd(7, H, seed=2)
    got = norm.forward(x.to(dtype).to(DEV))
    assert got.dtype == dtype
    assert torch.allclose(got.float().cpu(), P.plain_rms_norm(rounded(x, dtype), rounded(w, dtype), eps), **tol(dtype))
    # the fused form: the stream takes the branch, the norm is of the sum
    stream = rnd(7, H, seed=3).to(DEV)
    before = stream.clone()
    got = norm.forward_add(x.to(dtype).to(DEV), stream)
    want_stream = before.cpu() + rounded(x, dtype)
    assert torch.allclose(stream.cpu(), want_stream, atol=1e-6)
    assert torch.allclose(got.float().cpu(), P.plain_rms_norm(want_stream, rounded(w, dtype), eps), **tol(dtype))
    rows = torch.tensor([5, 0], dtype=torch.int32, device=DEV)
    picked = norm.forward_add(None, stream, rows=rows)
    assert torch.allclose(picked.float().cpu(), P.plain_rms_norm(want_stream[[5, 0]], rounded(w, dtype), eps), **tol(dtype))
    # Gemma's "w + 1" is a parameter of the same part
    plus = build_part("norm", PartSpec("rms_norm", {"size": H, "eps": eps, "weight_offset": 1.0}), "n", rt)
    give(plus, {"n.weight": w - 1.0}, torch.float32)
    assert torch.allclose(plus.forward(x.to(dtype).to(DEV)).float().cpu(),
                          P.plain_rms_norm(rounded(x, dtype), w, eps), **tol(dtype))


def test_rotary_part_table_is_the_plain_angles():
    rt = runtime(torch.float32, max_positions=300)
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    for scaling, theta, rot in ((None, 10000.0, 16), (sc, 500000.0, 32), (None, 1000.0, 24)):
        pe = build_part("position", PartSpec("rotary", {"head_dim": 32, "theta": theta, "rotary_dim": rot,
                                                        "scaling": scaling}), "x", rt)
        pe.load_weights(None)
        table, r, neox = pe.rotary_table()
        assert (r, neox, tuple(table.shape)) == (rot, True, (300, rot))
        ang = P.plain_rope_angles(list(range(300)), P.plain_rope_inv_freq(rot, theta, scaling))
        assert torch.allclose(table.cpu(), torch.cat([ang.cos(), ang.sin()], 1), atol=2e-6)
        # apply(): rotation alone, on a fused buffer of 3 q heads and 1 k head (v untouched)
        qkv = rnd(5, 5 * 32, seed=4)
        pos = [0, 7, 299, 64, 1]
        buf = qkv.clone().to(DEV)
        pe.apply(buf, 3, 1, 32, torch.tensor(pos, dtype=torch.int32, device=DEV))
        want = qkv.clone()
        want[:, :128] = P.plain_apply_rope(qkv[:, :128].view(5, 4, 32), pos, P.plain_rope_inv_freq(rot, theta, scaling),
                                           rotary_dim=rot).reshape(5, 128)
        assert torch.allclose(buf.cpu(), want, atol=1e-5)
    with pytest.raises(ValueError, match="rotary_dim"):
        build_part("position", PartSpec("rotary", {"head_dim": 32, "theta": 1e4, "rotary_dim": 34}), "x", rt)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_parts(dtype):
    rt = runtime(dtype)
    V, H = 331, 80
    table, head_w = rnd(V, H, seed=5), rnd(V, H, seed=6, scale=0.1)
    emb = build_part("embedding", PartSpec("token_embedding", {"vocab_size": V, "hidden_size": H, "scale": 2.0}), "e", rt)
    give(emb, {"e.weight": table}, dtype)
    ids = [330, 0, 17, 17]
    got = emb.forward(torch.tensor(ids, dtype=torch.int32, device=DEV))
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), rounded(table, dtype)[ids] * 2.0)
    head = build_part("head", PartSpec("lm_head", {"vocab_size": V, "hidden_size": H}), "lm_head", rt)
    give(head, {"lm_head.weight": head_w}, dtype)
    h = rnd(3, H, seed=7)
    logits = head.forward(h.to(dtype).to(DEV))
    assert logits.dtype == torch.float32 and logits.shape == (3, V)
    assert torch.allclose(logits.cpu(), P.plain_linear(rounded(h, dtype), rounded(head_w, dtype)), **tol(dtype))
    tied = build_part("head", PartSpec("lm_head", {"vocab_size": V, "hidden_size": H, "weight_name": "e.weight"}), "lm_head", rt)
    assert list(tied.checkpoint_tensors()) == ["e.weight"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bias", [False, True])
def test_gated_mlp_part(dtype, bias):
    rt = runtime(dtype)
    H, I = 80, 208
    ffn = build_part("feed_forward", PartSpec("gated_mlp", {"hidden_size": H, "intermediate_size": I, "bias": bias}), "m", rt)
    t = {"m.gate_proj.weight": rnd(I, H, seed=8, scale=0.2), "m.up_proj.weight": rnd(I, H, seed=9, scale=0.2),
         "m.down_proj.weight": rnd(H, I, seed=10, scale=0.2), "m.gate_proj.bias": rnd(I, seed=11),
         "m.up_proj.bias": rnd(I, seed=12), "m.down_proj.bias": rnd(H, seed=13)}
    want_names = {n for n in t if bias or not n.endswith(".bias")}
    decl = {}
    for p in ffn.walk():
        decl.update(p.checkpoint_tensors())
    assert set(decl) == want_names
    give(ffn, t, dtype)
    x = rnd(9, H, seed=14)
    r = {k: rounded(v, dtype) for k, v in t.items()}
    want = P.plain_swiglu_mlp(rounded(x, dtype), r["m.gate_proj.weight"], r["m.up_proj.weight"], r["m.down_proj.weight"],
                              *((r["m.gate_proj.bias"], r["m.up_proj.bias"], r["m.down_proj.bias"]) if bias else ()))
    got = ffn.forward(x.to(dtype).to(DEV))
    assert close(got, want, dtype), (got.float().cpu() - want).abs().max()


def attention_tensors(H, nh, nkv, d, seed):
    return {"a.q_proj.weight": rnd(nh * d, H, seed=seed, scale=0.3), "a.k_proj.weight": rnd(nkv * d, H, seed=seed + 1, scale=0.3),
            "a.v_proj.weight": rnd(nkv * d, H, seed=seed + 2, scale=0.3), "a.o_proj.weight": rnd(H, nh * d, seed=seed + 3, scale=0.3),
            "a.q_proj.bias": rnd(nh * d, seed=seed + 4), "a.k_proj.bias": rnd(nkv * d, seed=seed + 5),
            "a.v_proj.bias": rnd(nkv * d, seed=seed + 6), "a.o_proj.bias": rnd(H, seed=seed + 7)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,ps,window", [(4, 2, 16, 8, None), (6, 1, 32, 16, 21), (5, 5, 48, 4, None)])
def test_paged_attention_part(dtype, nh, nkv, d, ps, window):
    rt = runtime(dtype)
    H, T, first = 72, 45, 0
    spec = PartSpec("paged_attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                        "position": PartSpec("rotary", {"head_dim": d, "theta": 100.0}),
                                        "qkv_bias": True, "out_bias": True, "window": window})
    att = build_part("mixer", spec, "a", rt)
    assert att.cache_spec().num_kv_heads == nkv and att.cache_spec().window == window and att.state_spec() is None
    t = attention_tensors(H, nh, nkv, d, seed=20)
    give(att, t, dtype)
    ctx, n_pages = whole_prompt_context(T, ps, first_pos=first)
    binding = CacheBinding(group=0, k_pages=torch.zeros(n_pages, nkv, ps, d, dtype=dtype, device=DEV),
                           v_pages=torch.zeros(n_pages, nkv, d, ps, dtype=dtype, device=DEV))
    x = rnd(T, H, seed=30)
    got = att.forward(x.to(dtype).to(DEV), ctx, binding)
    r = {k: rounded(v, dtype) for k, v in t.items()}
    xr = rounded(x, dtype)
    inv = P.plain_rope_inv_freq(d, 100.0)
    pos = list(range(first, first + T))
    q = P.plain_apply_rope(P.plain_linear(xr, r["a.q_proj.weight"], r["a.q_proj.bias"]).view(T, nh, d), pos, inv)
    k = P.plain_apply_rope(P.plain_linear(xr, r["a.k_proj.weight"], r["a.k_proj.bias"]).view(T, nkv, d), pos, inv)
    v = P.plain_linear(xr, r["a.v_proj.weight"], r["a.v_proj.bias"]).view(T, nkv, d)
    a = P.plain_attention(q, k, v, window=window)
    want = P.plain_linear(a.reshape(T, nh * d), r["a.o_proj.weight"], r["a.o_proj.bias"])
    assert close(got, want, dtype), (got.float().cpu() - want).abs().max()
    # the keys and values lie in the pages at their slots: rotated keys, plain values
    kc = binding.k_pages.float().cpu().permute(0, 2, 1, 3).reshape(n_pages * ps, nkv, d)[first:first + T]
    vc = binding.v_pages.float().cpu().permute(0, 3, 1, 2).reshape(n_pages * ps, nkv, d)[first:first + T]
    assert torch.allclose(kc, k, **tol(dtype)) and torch.allclose(vc, v, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part_is_the_plain_layer(dtype, tmp_path):
    folder, cfg = make_model_folder(tmp_path, "B", dtype="float32")
    cfg_dict, w = P.read_model_folder(folder)
    rt = runtime(dtype, max_positions=cfg.max_position_embeddings)
    spec = build_llama_spec(cfg)
    ls = spec.layers[1]
    mixer = build_part("mixer", ls.mixer, ls.prefix + ".self_attn", rt)
    ffn = build_part("feed_forward", ls.feed_forward, ls.prefix + ".mlp", rt)
    norms = {role: build_part("norm", ns, ls.prefix + "." + ns.params["prefix"], rt) for role, ns in ls.norms.items()}
    block = build_part("block", ls.block, ls.prefix, rt, mixer=mixer, feed_forward=ffn, norms=norms)
    give(block, w, dtype)
    T, ps = 40, 16
    ctx, n_pages = whole_prompt_context(T, ps)
    nkv, d = cfg.num_key_value_heads, cfg.head_dim
    binding = CacheBinding(group=0, k_pages=torch.zeros(n_pages, nkv, ps, d, dtype=dtype, device=DEV),
                           v_pages=torch.zeros(n_pages, nkv, d, ps, dtype=dtype, device=DEV))
    stream0, branch0 = rnd(T, cfg.hidden_size, seed=40), rnd(T, cfg.hidden_size, seed=41, scale=0.1)
    stream = stream0.clone().to(DEV)
    out_branch = block.forward(branch0.to(dtype).to(DEV), stream, ctx, binding)
    wr = {k: rounded(v, dtype) for k, v in w.items()}
    inv = P.plain_rope_inv_freq(d, cfg_dict["rope_theta"], cfg_dict["rope_scaling"])
    want, _ = P.plain_llama_layer(cfg_dict, wr, ls.prefix, stream0 + rounded(branch0, dtype), list(range(T)), inv)
    # the block leaves its feed-forward output to be added by the next norm
    got = stream.cpu() + out_branch.float().cpu()
    assert torch.allclose(got, want, **tol(dtype)), (got - want).abs().max()
    with pytest.raises(ValueError, match="needs norms"):
        build_part("block", ls.block, ls.prefix, rt, mixer=mixer, feed_forward=ffn, norms={"input": norms["input"]})


# --------------------------------------------------------------------------- the same parts, arranged differently

class VariantConfig(LlamaConfig):
    ARCHITECTURE = "VariantForCausalLM"
    MODEL_TYPE = "variant"


VARIANT_SCHEDULE = [(0, None), (1, None), (2, 1), (0, None)]     # layer 0 runs twice; layer 2 reads layer 1's cache
VARIANT_WINDOWS = {0: 40}                                         # both runs of layer 0 see the last 40 keys only


def build_variant_spec(cfg):
    base = build_llama_spec(cfg)
    layers = tuple(
        LayerSpec(prefix=ls.prefix, block=ls.block, feed_forward=ls.feed_forward, norms=ls.norms,
                  mixer=ls.mixer.with_params(window=VARIANT_WINDOWS[i]) if i in VARIANT_WINDOWS else ls.mixer)
        for i, ls in enumerate(base.layers))
    return ModelSpec(embedding=base.embedding, layers=layers,
                     schedule=tuple(ScheduleEntry(l, src) for l, src in VARIANT_SCHEDULE),
                     final_norm=base.final_norm, head=base.head, vocab_size=base.vocab_size, hidden_size=base.hidden_size)


@pytest.fixture
def variant_architecture():
    register_architecture("VariantForCausalLM", "variant", VariantConfig, build_variant_spec)
    yield
    unregister_architecture("VariantForCausalLM")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_twice_shared_cache_and_window(variant_architecture, tmp_path, dtype):
    from test_replay_gpu import check, spike_far_key, tolerance
    cfg = VariantConfig.from_dict(dict(TINY_B, torch_dtype=dtype))
    folder = write_random_model(str(tmp_path / "variant"), cfg, seed=4, dtype=dtype)
    # layer 0 is made to attend to the key of token 5 wherever it stands, so that the window's edge shows:
    # 40 positions after that token the logits change
    folder = spike_far_key(folder, P.read_model_folder(folder)[0])
    cfg_dict, w = P.read_model_folder(folder)
    clean = lambda toks: [t if t != 5 else 6 for t in toks]
    reqs = {"a": clean(random_tokens(150, cfg.vocab_size, 1)), "b": clean(random_tokens(41, cfg.vocab_size, 2)),
            "c": clean(random_tokens(97, cfg.vocab_size, 3)), "d": clean(random_tokens(40, cfg.vocab_size, 4))}
    reqs["a"][18] = 5
    reqs["c"][50] = 5
    refs = {r: P.plain_llama_forward(cfg_dict, w, toks, schedule=VARIANT_SCHEDULE, windows=VARIANT_WINDOWS)
            for r, toks in reqs.items()}
    no_window = P.plain_llama_forward(cfg_dict, w, reqs["a"], schedule=VARIANT_SCHEDULE)
    assert (no_window[:40] - refs["a"][:40]).abs().max() < 1e-4                       # shorter than the window: the same
    assert (no_window[58:] - refs["a"][58:]).abs().max() > 5 * tolerance(dtype, refs["a"])  # the marked key has left it
    core = load_engine_core(folder, dtype=dtype, block_size=16, num_pages=20, max_num_seqs=4)
    assert [g.spec.window for g in core.storage.groups] == [40, None]                 # a pool of pages for each need
    assert core.storage.entry_group == [0, 1, 1, 0]
    assert [b.writes_cache for b in core.storage.bindings] == [True, True, False, True]
    assert core.storage.bindings[2].k_pages is core.storage.bindings[1].k_pages
    assert core.storage.bindings[3].k_pages is not core.storage.bindings[0].k_pages
    for name, steps in (("whole", trace_whole(reqs)), ("bulk then single", trace_bulk_then_single(reqs)),
                        ("portions", trace_portions(reqs, seed=3)), ("mixed", trace_mixed(reqs, 320, seed=2))):
        check(replay_in_process(core.executor, steps), refs, dtype, name)
        core.storage.manager.check_invariants()
        assert [core.storage.manager.num_free_pages(g) for g in (0, 1)] == [20, 20]
    # while a long request is held, the window group keeps only the pages the window still covers
    ex = core.executor
    ex.step([StepEntry("long", reqs["a"], [])])
    assert 20 - core.storage.manager.num_free_pages(1) == 10 and 20 - core.storage.manager.num_free_pages(0) <= 4
    ex.release("long")


# --------------------------------------------------------------------------- toy parts, defined here

class RunningMeanMixer(Mixer):
    """out[t] = W mean(h[0..t]) over the request's tokens so far. Its state (the running sum and the count)
    is fixed-size per request and lives in the state slots; it has no paged cache."""

    def __init__(self, prefix, rt, hidden_size):
        super().__init__(prefix, rt)
        self.H = hidden_size
        self.weight = None

    def checkpoint_tensors(self):
        return {self.prefix + ".weight": TensorDecl((self.H, self.H))}

    def load_weights(self, fetch):
        self.weight = fetch(self.prefix + ".weight")

    def state_spec(self):
        return StateSpec((self.H + 1,), torch.float32)

    def forward(self, h, ctx, binding):
        out = torch.empty_like(h)
        for s, (start, n, first, slot) in enumerate(zip(ctx.host_seg_starts, ctx.host_seg_lens, ctx.host_seg_first_pos,
                                                        ctx.host_state_slots)):
            st = binding.state[slot]                              # (all zeros when a request begins: the engine clears it)
            x = h[start:start + n].float()
            sums = st[:self.H] + torch.cumsum(x, 0)
            counts = st[self.H] + torch.arange(1, n + 1, device=h.device, dtype=torch.float32)
            out[start:start + n] = ((sums / counts[:, None]) @ self.weight.float().t()).to(h.dtype)
            st[:self.H] = sums[-1]
            st[self.H] = counts[-1]
        return out


class RoutedFeedForward(FeedForward):
    """Every token goes to the expert with the largest router logit (float32), scaled by its softmax weight."""

    def __init__(self, prefix, rt, hidden_size, intermediate_size, num_experts):
        super().__init__(prefix, rt)
        self.H, self.I, self.E = hidden_size, intermediate_size, num_experts

    def checkpoint_tensors(self):
        out = {self.prefix + ".router.weight": TensorDecl((self.E, self.H))}
        for e in range(self.E):
            out["%s.experts.%d.up.weight" % (self.prefix, e)] = TensorDecl((self.I, self.H))
            out["%s.experts.%d.down.weight" % (self.prefix, e)] = TensorDecl((self.H, self.I))
        return out

    def load_weights(self, fetch):
        self.router = fetch(self.prefix + ".router.weight")
        self.up = [fetch("%s.experts.%d.up.weight" % (self.prefix, e)) for e in range(self.E)]
        self.down = [fetch("%s.experts.%d.down.weight" % (self.prefix, e)) for e in range(self.E)]

    def forward(self, h):
        logits = h.float() @ self.router.float().t()
        gate, choice = torch.softmax(logits, -1).max(-1)
        out = torch.zeros_like(h, dtype=torch.float32)
        for e in range(self.E):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel():
                x = h[rows].float()
                out[rows] = torch.relu(x @ self.up[e].float().t()) @ self.down[e].float().t() * gate[rows, None]
        return out.to(h.dtype)


class LearnedPositions(PositionEncoding):
    """Adds a learned vector per position to every query and key head (no rotation)."""

    def __init__(self, prefix, rt, head_dim):
        super().__init__(prefix, rt)
        self.d = head_dim

    def checkpoint_tensors(self):
        return {self.prefix + ".positions": TensorDecl((self.rt.max_positions, self.d))}

    def load_weights(self, fetch):
        self.table = fetch(self.prefix + ".positions")

    def apply(self, qkv, nh, nkv, d, positions):
        add = self.table[positions.long()].to(qkv.dtype)
        heads = qkv[:, :(nh + nkv) * d].view(qkv.shape[0], nh + nkv, d)
        heads += add[:, None, :]


class ToyConfig(LlamaConfig):
    ARCHITECTURE = "ToyForCausalLM"
    MODEL_TYPE = "toy"


def build_toy_spec(cfg):
    H = cfg.hidden_size

    def norm(prefix):
        return PartSpec("rms_norm", {"prefix": prefix, "size": H, "eps": cfg.rms_norm_eps})

    norms = {"input": norm("ln1"), "post_mixer": norm("ln2")}
    stateful = LayerSpec("toy.layers.0", PartSpec("prenorm_residual"),
                         PartSpec("toy_running_mean", {"prefix": "mean", "hidden_size": H}),
                         PartSpec("toy_routed", {"prefix": "moe", "hidden_size": H, "intermediate_size": cfg.intermediate_size,
                                                 "num_experts": 3}), norms)
    attending = LayerSpec("toy.layers.1", PartSpec("prenorm_residual"),
                          PartSpec("paged_attention", {"prefix": "attn", "hidden_size": H, "num_heads": cfg.num_attention_heads,
                                                       "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                                                       "position": PartSpec("toy_learned_positions", {"head_dim": cfg.head_dim})}),
                          PartSpec("gated_mlp", {"prefix": "mlp", "hidden_size": H, "intermediate_size": cfg.intermediate_size}),
                          norms)
    return ModelSpec(
        embedding=PartSpec("token_embedding", {"prefix": "toy.embed", "vocab_size": cfg.vocab_size, "hidden_size": H}),
        layers=(stateful, attending), schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)),
        final_norm=norm("toy.norm"), head=PartSpec("lm_head", {"prefix": "toy.head", "vocab_size": cfg.vocab_size,
                                                               "hidden_size": H}),
        vocab_size=cfg.vocab_size, hidden_size=H)


def plain_toy_forward(cfg, w, toks):
    """The toy model on a whole sequence, float32, nothing shared with the parts above."""
    H, nh, nkv, d, eps = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps
    T = len(toks)
    s = P.plain_embedding(w["toy.embed.weight"], toks)

    def stateful(s):
        p = "toy.layers.0."
        h = P.plain_rms_norm(s, w[p + "ln1.weight"], eps)
        mean = torch.stack([h[:t + 1].mean(0) for t in range(T)])
        s = s + P.plain_linear(mean, w[p + "mean.weight"])
        h = P.plain_rms_norm(s, w[p + "ln2.weight"], eps)
        probs = torch.softmax(P.plain_linear(h, w[p + "moe.router.weight"]), -1)
        out = torch.zeros(T, H)
        for t in range(T):
            e = int(probs[t].argmax())
            up = torch.relu(P.plain_linear(h[t:t + 1], w[p + "moe.experts.%d.up.weight" % e]))
            out[t] = P.plain_linear(up, w[p + "moe.experts.%d.down.weight" % e])[0] * probs[t, e]
        return s + out

    s = stateful(s)
    p = "toy.layers.1."
    h = P.plain_rms_norm(s, w[p + "ln1.weight"], eps)
    add = w[p + "attn.positions"][:T]
    q = P.plain_linear(h, w[p + "attn.q_proj.weight"]).view(T, nh, d) + add[:, None]
    k = P.plain_linear(h, w[p + "attn.k_proj.weight"]).view(T, nkv, d) + add[:, None]
    v = P.plain_linear(h, w[p + "attn.v_proj.weight"]).view(T, nkv, d)
    s = s + P.plain_linear(P.plain_attention(q, k, v).reshape(T, nh * d), w[p + "attn.o_proj.weight"])
    h = P.plain_rms_norm(s, w[p + "ln2.weight"], eps)
    s = s + P.plain_swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    s = stateful(s)                                              # the first layer again, with state of its own
    return P.plain_linear(P.plain_rms_norm(s, w["toy.norm.weight"], eps), w["toy.head.weight"])


@pytest.fixture
def toy_architecture():
    register_part("mixer", "toy_running_mean")(RunningMeanMixer)
    register_part("feed_forward", "toy_routed")(RoutedFeedForward)
    register_part("position", "toy_learned_positions")(LearnedPositions)
    register_architecture("ToyForCausalLM", "toy", ToyConfig, build_toy_spec)
    yield
    unregister_architecture("ToyForCausalLM")
    unregister_part("mixer", "toy_running_mean")
    unregister_part("feed_forward", "toy_routed")
    unregister_part("position", "toy_learned_positions")


def test_toy_parts_are_registered_built_and_stepped(toy_architecture, tmp_path):
    cfg = ToyConfig.from_dict(dict(TINY["A"][0], tie_word_embeddings=False, max_position_embeddings=96))
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=9, std=0.3)
    _, w = P.read_model_folder(folder)
    assert "toy.layers.0.moe.experts.2.down.weight" in w and "toy.layers.1.attn.positions" in w
    core = load_engine_core(folder, dtype="float32", block_size=8, num_pages=24, max_num_seqs=3)
    reqs = {"a": random_tokens(50, cfg.vocab_size, 1), "b": random_tokens(9, cfg.vocab_size, 2),
            "c": random_tokens(33, cfg.vocab_size, 3), "d": random_tokens(64, cfg.vocab_size, 4),
            "e": random_tokens(21, cfg.vocab_size, 5)}
    refs = {r: plain_toy_forward(cfg, w, toks) for r, toks in reqs.items()}
    used = {int(torch.softmax(P.plain_linear(P.plain_rms_norm(P.plain_embedding(w["toy.embed.weight"], reqs["d"]),
                                                              w["toy.layers.0.ln2.weight"], cfg.rms_norm_eps),
                                             w["toy.layers.0.moe.router.weight"]), -1)[t].argmax()) for t in range(64)}
    assert len(used) > 1                                         # the routing does route
    # the two runs of layer 0 have a state tensor each, one slot per live request and a spare one; no pages for them
    states = [b.state for b in core.storage.bindings]
    assert states[0] is not None and states[2] is not None and states[1] is None
    assert states[0].data_ptr() != states[2].data_ptr() and tuple(states[0].shape) == (3 + 1, cfg.hidden_size + 1)
    assert core.storage.entry_group == [None, 0, None]
    assert not core.executor.use_graphs                          # a part that does not declare itself graph-safe: eager
    # the step is a recorded program all the same: the parts the recorder cannot follow (the two runs of the mean
    # mixer and of the routed feed-forward, the learned positions) are five callbacks in it, the rest is native
    prog = core.executor.program
    assert prog is not None and len(prog.callbacks) == 5, [c.what for c in prog.callbacks] if prog else None
    from test_replay_gpu import check
    for name, steps in (("whole", trace_whole(reqs)), ("bulk then single", trace_bulk_then_single(reqs)),
                        ("portions", trace_portions(reqs, seed=7)),
                        ("mixed", trace_mixed(reqs, 192, seed=3, max_live=3))):      # 5 requests through 3 state slots
        check(replay_in_process(core.executor, steps), refs, "float32", name)
        assert core.storage.manager.num_free_state_slots() == 3
    assert core.executor.program_steps > 50
    # part by part, without the program: the same bits
    plain = load_engine_core(folder, dtype="float32", block_size=8, num_pages=24, max_num_seqs=3, use_program=False)
    steps = trace_mixed(reqs, 192, seed=3, max_live=3)
    a, b = replay_in_process(core.executor, steps), replay_in_process(plain.executor, steps)
    assert plain.executor.program is None and all(torch.equal(a[r], b[r]) for r in a)
    # bfloat16 builds and steps too
    core16 = load_engine_core(folder, dtype="bfloat16", block_size=8, num_pages=24, max_num_seqs=3)
    out = core16.executor.step([StepEntry("x", reqs["b"], [len(reqs["b"]) - 1])])
    check({"x": out.float().cpu()}, {"x": refs["b"][-1:]}, "bfloat16", "toy parts in bfloat16")


# --------------------------------------------------------------------------- a mixer whose values are wider than its keys

class WideValueAttention(Mixer):
    """Causal attention with keys of width d and values of width dv, written with torch: it stores into its pages
    and reads from them through the block tables itself (the package's kernels take equal widths)."""

    def __init__(self, prefix, rt, hidden_size, num_heads, num_kv_heads, head_dim, v_head_dim):
        super().__init__(prefix, rt)
        self.H, self.nh, self.nkv, self.d, self.dv = hidden_size, num_heads, num_kv_heads, head_dim, v_head_dim

    def _shapes(self):
        return {"q": (self.nh * self.d, self.H), "k": (self.nkv * self.d, self.H), "v": (self.nkv * self.dv, self.H),
                "o": (self.H, self.nh * self.dv)}

    def checkpoint_tensors(self):
        return {"%s.%s.weight" % (self.prefix, n): TensorDecl(s) for n, s in self._shapes().items()}

    def load_weights(self, fetch):
        self.w = {n: fetch("%s.%s.weight" % (self.prefix, n)) for n in self._shapes()}

    def tensors(self):
        return list(self.w.values())

    def cache_spec(self):
        from lmsf_amd.parts import CacheSpec
        return CacheSpec(num_kv_heads=self.nkv, head_dim=self.d, v_head_dim=self.dv)

    def forward(self, h, ctx, binding):
        N = h.shape[0]
        x = h.float()
        q = (x @ self.w["q"].float().t()).view(N, self.nh, self.d)
        k = (x @ self.w["k"].float().t()).view(N, self.nkv, self.d)
        v = (x @ self.w["v"].float().t()).view(N, self.nkv, self.dv)
        group = ctx.groups[binding.group]
        ps = group.page_size
        slots = group.slots.long()
        binding.k_pages[slots // ps, :, slots % ps, :] = k.to(binding.k_pages.dtype)
        binding.v_pages[slots // ps, :, :, slots % ps] = v.to(binding.v_pages.dtype)
        out = torch.empty(N, self.nh, self.dv, dtype=torch.float32, device=h.device)
        rep = self.nh // self.nkv
        for s, (start, n, first) in enumerate(zip(ctx.host_seg_starts, ctx.host_seg_lens, ctx.host_seg_first_pos)):
            T = first + n
            pages = group.block_tables[s, :-(-T // ps)].long()
            K = binding.k_pages[pages].float().permute(1, 0, 2, 3).reshape(self.nkv, -1, self.d)[:, :T]
            V = binding.v_pages[pages].float().permute(1, 0, 3, 2).reshape(self.nkv, -1, self.dv)[:, :T]
            qs = q[start:start + n]
            scores = torch.einsum("thd,hjd->thj", qs, K.repeat_interleave(rep, 0)) / self.d ** 0.5
            dead = torch.arange(T, device=h.device)[None, :] > (first + torch.arange(n, device=h.device))[:, None]
            probs = torch.softmax(scores.masked_fill(dead[:, None, :], float("-inf")), -1)
            out[start:start + n] = torch.einsum("thj,hjd->thd", probs, V.repeat_interleave(rep, 0))
        return (out.reshape(N, self.nh * self.dv) @ self.w["o"].float().t()).to(h.dtype)


class WideConfig(LlamaConfig):
    ARCHITECTURE = "WideValueForCausalLM"
    MODEL_TYPE = "wide_value"


WIDE_DV = 24      # values of 24 numbers beside keys of 16


def build_wide_spec(cfg):
    H = cfg.hidden_size

    def norm(prefix):
        return PartSpec("rms_norm", {"prefix": prefix, "size": H, "eps": cfg.rms_norm_eps})

    layers = tuple(LayerSpec("wide.layers.%d" % i, PartSpec("prenorm_residual"),
                             PartSpec("toy_wide_value", {"prefix": "attn", "hidden_size": H, "num_heads": cfg.num_attention_heads,
                                                         "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                                                         "v_head_dim": WIDE_DV}),
                             PartSpec("gated_mlp", {"prefix": "mlp", "hidden_size": H, "intermediate_size": cfg.intermediate_size}),
                             {"input": norm("ln1"), "post_mixer": norm("ln2")}) for i in range(cfg.num_hidden_layers))
    return ModelSpec(
        embedding=PartSpec("token_embedding", {"prefix": "wide.embed", "vocab_size": cfg.vocab_size, "hidden_size": H}),
        layers=layers, schedule=tuple(ScheduleEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=norm("wide.norm"), head=PartSpec("lm_head", {"prefix": "wide.head", "vocab_size": cfg.vocab_size,
                                                                "hidden_size": H}),
        vocab_size=cfg.vocab_size, hidden_size=H)


def plain_wide_forward(cfg, w, toks):
    H, nh, nkv, d, eps = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps
    T = len(toks)
    s = P.plain_embedding(w["wide.embed.weight"], toks)
    for i in range(cfg.num_hidden_layers):
        p = "wide.layers.%d." % i
        h = P.plain_rms_norm(s, w[p + "ln1.weight"], eps)
        q = P.plain_linear(h, w[p + "attn.q.weight"]).view(T, nh, d)
        k = P.plain_linear(h, w[p + "attn.k.weight"]).view(T, nkv, d)
        v = P.plain_linear(h, w[p + "attn.v.weight"]).view(T, nkv, WIDE_DV)
        s = s + P.plain_linear(P.plain_attention(q, k, v).reshape(T, nh * WIDE_DV), w[p + "attn.o.weight"])
        h = P.plain_rms_norm(s, w[p + "ln2.weight"], eps)
        s = s + P.plain_swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.plain_linear(P.plain_rms_norm(s, w["wide.norm.weight"], eps), w["wide.head.weight"])


def test_a_mixer_with_values_wider_than_its_keys(tmp_path):
    """A cache group may hold values of another width than its keys (CacheSpec.v_head_dim): the pages are made so,
    a page's bytes count both widths, and a toy mixer that reads and writes such pages itself goes through the
    four ways of cutting, with pages used again, as a callback inside the recorded program."""
    register_part("mixer", "toy_wide_value")(WideValueAttention)
    register_architecture("WideValueForCausalLM", "wide_value", WideConfig, build_wide_spec)
    try:
        cfg = WideConfig.from_dict(dict(TINY["A"][0], tie_word_embeddings=False, max_position_embeddings=96))
        folder = write_random_model(str(tmp_path / "wide"), cfg, seed=4, std=0.2)
        _, w = P.read_model_folder(folder)
        core = load_engine_core(folder, dtype="float32", block_size=8, num_pages=24, max_num_seqs=4)
        b = core.storage.bindings[0]
        assert tuple(b.k_pages.shape) == (24, cfg.num_key_value_heads, 8, cfg.head_dim)
        assert tuple(b.v_pages.shape) == (24, cfg.num_key_value_heads, WIDE_DV, 8)
        assert core.storage.groups[0].bytes_per_page(4) == 2 * cfg.num_key_value_heads * 8 * (cfg.head_dim + WIDE_DV) * 4
        prog = core.executor.program
        assert prog is not None and len(prog.callbacks) == cfg.num_hidden_layers
        reqs = {"a": random_tokens(50, cfg.vocab_size, 1), "b": random_tokens(9, cfg.vocab_size, 2),
                "c": random_tokens(33, cfg.vocab_size, 3), "d": random_tokens(64, cfg.vocab_size, 4),
                "e": random_tokens(21, cfg.vocab_size, 5)}
        refs = {r: plain_wide_forward(cfg, w, toks) for r, toks in reqs.items()}
        from test_replay_gpu import check
        for name, steps in (("whole", trace_whole(reqs)), ("bulk then single", trace_bulk_then_single(reqs)),
                            ("portions", trace_portions(reqs, seed=7)), ("mixed", trace_mixed(reqs, 192, seed=3))):
            check(replay_in_process(core.executor, steps), refs, "float32", "wide values, " + name)
            assert core.storage.manager.num_free_pages(0) == 24
    finally:
        unregister_architecture("WideValueForCausalLM")
        unregister_part("mixer", "toy_wide_value")
