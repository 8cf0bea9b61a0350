"""What fixes the plain implementation beside the reference's text.

The reference's own tests hold inputs without expected outputs (tops/src/rms_norm.rs:100-130 prints
its result; tops/csrc/example/test_softmax.cc prints too), so no vector pins a formula. Each
function of plain_llama is therefore pinned by a special case that reduces to a library routine
and by invariants, each chosen so that a plausible mistake fails it: a wrong sign or pairing in
the rotation, eps outside the root, a norm in the wrong place, the wrong kv head for a query head,
gate and up swapped. The sampler's parity with the reference is unpinned beyond its text.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
from helpers import make_model_folder, random_tokens


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


# --------------------------------------------------------------------------- RMSNorm

def test_rms_norm_is_the_library_routine():
    x, w = rnd(5, 48, seed=1), rnd(48, seed=2)
    for eps in (1e-5, 1e-6, 0.3):
        assert torch.allclose(P.plain_rms_norm(x, w, eps), F.rms_norm(x, (48,), w, eps), atol=1e-6)


def test_rms_norm_eps_is_under_the_root_and_mean_is_over_the_row():
    # the input of the reference's own test (tops/src/rms_norm.rs:103-120), rows of 2 as there
    a = torch.tensor([-0.16046895, -1.03667831, -0.34974465, 0.26505867, -1.24111986, -0.53806001, 1.72426331,
                      0.43572459, -0.77390957, -0.42610624, 0.16398858, -1.35760343, 1.07541728, 0.11008703,
                      0.26361224, -0.48663723]).reshape(8, 2)
    y = P.plain_rms_norm(a, torch.ones(2), 1e-5)
    for r in range(8):
        ms = (a[r, 0] ** 2 + a[r, 1] ** 2) / 2
        assert torch.allclose(y[r], a[r] / math.sqrt(ms + 1e-5), atol=1e-6)
    # a tiny row: eps dominates, so eps outside the root or added to the sum instead of the mean shows
    x = torch.tensor([[1e-4, -2e-4, 3e-4, 0.0]])
    want = x / math.sqrt((1e-8 + 4e-8 + 9e-8) / 4 + 1e-2)
    assert torch.allclose(P.plain_rms_norm(x, torch.ones(4), 1e-2), want, rtol=1e-5, atol=0)


def test_rms_norm_invariants():
    x, w = rnd(3, 64, seed=3), torch.ones(64)
    y = P.plain_rms_norm(x, w, 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(3), atol=1e-5)          # unit mean square
    assert torch.allclose(P.plain_rms_norm(7.0 * x, w, 1e-12), y, atol=1e-5)   # scale does not matter
    assert torch.allclose(P.plain_rms_norm(x[1:2], w, 1e-6), P.plain_rms_norm(x, w, 1e-6)[1:2])  # rows independent
    w2 = rnd(64, seed=4)
    assert torch.allclose(P.plain_rms_norm(x, w2, 1e-6), P.plain_rms_norm(x, w, 1e-6) * w2, atol=1e-6)  # w, not 1 + w


# --------------------------------------------------------------------------- rotary

def test_rope_frequencies_closed_form():
    inv = P.plain_rope_inv_freq(32, 10000.0)      # the table parameters of vllm/src/pos_encoding.rs:48-56
    assert inv.shape == (16,)
    for i in (0, 1, 7, 15):
        assert abs(inv[i].item() - 10000.0 ** (-2.0 * i / 32)) < 1e-7
    assert inv[0].item() == 1.0


def test_rope_single_pair_is_a_rotation_by_position_times_frequency():
    d = 8
    inv = P.plain_rope_inv_freq(d, 100.0)
    for i in range(d // 2):
        x = torch.zeros(1, 1, d)
        x[0, 0, i] = 1.0                          # one-hot probe in the first half
        y = P.plain_apply_rope(x, [3], inv)[0, 0]
        ang = 3.0 * inv[i].item()
        want = torch.zeros(d)
        want[i], want[i + d // 2] = math.cos(ang), math.sin(ang)      # NeoX: partner is i + d/2; sign of sin +
        assert torch.allclose(y, want, atol=1e-6), (i, y)
        x = torch.zeros(1, 1, d)
        x[0, 0, i + d // 2] = 1.0                 # one-hot in the second half
        y = P.plain_apply_rope(x, [3], inv)[0, 0]
        want = torch.zeros(d)
        want[i], want[i + d // 2] = -math.sin(ang), math.cos(ang)
        assert torch.allclose(y, want, atol=1e-6), (i, y)
    # GPT-J style pairs (2i, 2i+1)
    x = torch.zeros(1, 1, d)
    x[0, 0, 2] = 1.0
    y = P.plain_apply_rope(x, [5], inv, neox=False)[0, 0]
    want = torch.zeros(d)
    want[2], want[3] = math.cos(5.0 * inv[1].item()), math.sin(5.0 * inv[1].item())
    assert torch.allclose(y, want, atol=1e-6)


def test_rope_invariants():
    d, T = 16, 6
    inv = P.plain_rope_inv_freq(d, 10000.0)
    q, k = rnd(T, 2, d, seed=5), rnd(T, 2, d, seed=6)
    assert torch.equal(P.plain_apply_rope(q[:1], [0], inv), q[:1])              # position 0 is the identity
    r = P.plain_apply_rope(q, list(range(T)), inv)
    half = d // 2
    assert torch.allclose(r[..., :half] ** 2 + r[..., half:] ** 2, q[..., :half] ** 2 + q[..., half:] ** 2, atol=1e-5)
    # <rope(q, m), rope(k, n)> depends on m - n only
    def dot(m, n):
        a = P.plain_apply_rope(q[:1], [m], inv)
        b = P.plain_apply_rope(k[:1], [n], inv)
        return (a * b).sum(-1)
    assert torch.allclose(dot(9, 4), dot(105, 100), atol=1e-4)
    assert torch.allclose(dot(5, 0), dot(40, 35), atol=1e-4)
    assert not torch.allclose(dot(9, 4), dot(9, 5), atol=1e-4)
    # partial rotation leaves the tail alone
    pr = P.plain_apply_rope(q, list(range(T)), P.plain_rope_inv_freq(8, 10000.0), rotary_dim=8)
    assert torch.equal(pr[..., 8:], q[..., 8:]) and not torch.allclose(pr[1:, :, :8], q[1:, :, :8])


def test_rope_llama3_scaling():
    base = P.plain_rope_inv_freq(64, 500000.0)
    same = P.plain_rope_inv_freq(64, 500000.0, dict(rope_type="llama3", factor=1.0, low_freq_factor=1.0,
                                                     high_freq_factor=4.0, original_max_position_embeddings=64))
    assert torch.allclose(base, same, rtol=1e-6)                                 # factor 1 changes nothing
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    f = P.plain_rope_inv_freq(64, 500000.0, sc)
    wavelen = 2 * math.pi / base
    hi, lo = wavelen < 64 / 4.0, wavelen > 64 / 1.0
    assert hi.any() and lo.any() and (~hi & ~lo).any()                           # all three regimes occur
    assert torch.equal(f[hi], base[hi])                                          # short waves are kept
    assert torch.allclose(f[lo], base[lo] / 8.0, rtol=1e-6)                      # long waves slowed by the factor
    mid = ~hi & ~lo
    ratio = (f / base)[mid]
    assert ((ratio > 1 / 8.0) & (ratio < 1.0)).all()
    assert (ratio[:-1] >= ratio[1:]).all()                                       # a monotone blend
    assert torch.equal(P.plain_rope_inv_freq(64, 500000.0, {"rope_type": "default"}), base)


def test_rope_llama3_blend_is_linear_in_frequency_and_meets_both_ends():
    """The band between the two wavelengths pinned by arithmetic alone: at the band's short end (wavelength
    orig / high) the blend is the frequency itself, at its long end (orig / low) the frequency over the factor,
    and at the frequency midway between the two ends the ratio is (1 + 1 / factor) / 2: the blend is linear in the
    frequency (a blend linear in the wavelength gives (1 + 1 / factor) / 2 midway between the wavelengths instead,
    and 0.4 here). With rotary_dim 4 the second frequency is theta^(-1/2), so theta places it anywhere. The same
    for the product's table builder."""
    from lmsf_amd.parts.rotary import inverse_frequencies
    orig, low, high, factor = 64.0, 1.0, 4.0, 8.0
    sc = dict(rope_type="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high,
              original_max_position_embeddings=int(orig))
    f_short, f_long = 2 * math.pi * high / orig, 2 * math.pi * low / orig
    cases = [(f_short, 1.0), (f_long, 1.0 / factor), ((f_short + f_long) / 2, (1 + 1 / factor) / 2),
             (f_long + 0.25 * (f_short - f_long), 0.25 + 0.75 / factor),
             (f_short * 1.5, 1.0), (f_long / 1.5, 1.0 / factor)]
    for f, want in cases:
        theta = 1.0 / (f * f)
        for build in (P.plain_rope_inv_freq, inverse_frequencies):
            got = build(4, theta, sc)
            assert got[0].item() == 1.0                              # wavelength 2 pi: short, kept
            assert abs(got[1].item() / f - want) < 2e-6, (build.__name__, f, got[1].item() / f, want)
    # what a blend linear in the wavelength would give midway between the frequencies: far from the above
    lam = 2 * math.pi / ((f_short + f_long) / 2)
    s_wave = (orig / low - lam) / (orig / low - orig / high)
    assert abs(((1 - s_wave) / factor + s_wave) - (1 + 1 / factor) / 2) > 0.05


# --------------------------------------------------------------------------- attention

@pytest.mark.parametrize("nh,nkv", [(4, 4), (4, 2), (6, 1)])
def test_attention_is_the_library_routine(nh, nkv):
    T, d = 9, 16
    q, k, v = rnd(T, nh, d, seed=7), rnd(T, nkv, d, seed=8), rnd(T, nkv, d, seed=9)
    got = P.plain_attention(q, k, v)
    kk = k.repeat_interleave(nh // nkv, dim=1).transpose(0, 1)     # kv head g serves heads g*n_rep .. g*n_rep+n_rep-1
    vv = v.repeat_interleave(nh // nkv, dim=1).transpose(0, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, is_causal=True).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-5)


def test_attention_without_mask_or_rotation_one_head():
    # last row of a causal attention sees every key: softmax(q K^T / sqrt d) V by library routines
    T, d = 7, 8
    q, k, v = rnd(T, 1, d, seed=10), rnd(T, 1, d, seed=11), rnd(T, 1, d, seed=12)
    got = P.plain_attention(q, k, v)[-1, 0]
    want = torch.softmax(q[-1, 0] @ k[:, 0].t() / math.sqrt(d), -1) @ v[:, 0]
    assert torch.allclose(got, want, atol=1e-6)


def test_attention_invariants():
    T, nh, nkv, d = 8, 4, 2, 16
    q, k, v = rnd(T, nh, d, seed=13), rnd(T, nkv, d, seed=14), rnd(T, nkv, d, seed=15)
    out = P.plain_attention(q, k, v)
    assert torch.allclose(out[0], v[0].repeat_interleave(2, dim=0), atol=1e-6)       # one key: its value
    same_k = k[:1].expand(T, nkv, d)
    mean_v = torch.cumsum(v, 0) / torch.arange(1, T + 1)[:, None, None]
    assert torch.allclose(P.plain_attention(q, same_k, v), mean_v.repeat_interleave(2, dim=1), atol=1e-5)
    k2, v2 = k.clone(), v.clone()
    k2[5:], v2[5:] = 9.0, -3.0                                                       # later tokens change nothing earlier
    assert torch.equal(P.plain_attention(q, k2, v2)[:5], out[:5])
    # a window of W keeps keys i-W+1 .. i
    w = P.plain_attention(q, k, v, window=3)
    assert torch.allclose(w[:3], out[:3], atol=1e-6)
    assert torch.allclose(w[6], P.plain_attention(q[4:7], k[4:7], v[4:7])[2], atol=1e-6)
    assert torch.allclose(P.plain_attention(q, k, v, scale=0.0), mean_v.repeat_interleave(2, dim=1), atol=1e-5)


# --------------------------------------------------------------------------- feed-forward, linear, embedding

def test_swiglu_is_library_routines_and_gate_comes_first():
    x, wg, wu, wd = rnd(5, 12, seed=16), rnd(20, 12, seed=17), rnd(20, 12, seed=18), rnd(12, 20, seed=19)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(P.plain_swiglu_mlp(x, wg, wu, wd), want, atol=1e-5)
    assert not torch.allclose(P.plain_swiglu_mlp(x, wu, wg, wd), want, atol=1e-3)     # swapped halves differ
    assert torch.equal(P.plain_swiglu_mlp(x, wg, torch.zeros_like(wu), wd), torch.zeros(5, 12))
    assert P.plain_silu(torch.zeros(3)).abs().max() == 0
    assert torch.allclose(P.plain_silu(torch.tensor([1.0, -2.0])), F.silu(torch.tensor([1.0, -2.0])), atol=1e-7)


def test_linear_and_embedding():
    x, w, b = rnd(4, 10, seed=20), rnd(6, 10, seed=21), rnd(6, seed=22)
    assert torch.allclose(P.plain_linear(x, w, b), F.linear(x, w, b), atol=1e-6)
    assert torch.equal(P.plain_linear(torch.zeros(2, 10), w, b), b.expand(2, 6))
    onehot = torch.zeros(1, 10)
    onehot[0, 3] = 1.0
    assert torch.equal(P.plain_linear(onehot, w)[0], w[:, 3])
    table = rnd(9, 5, seed=23)
    assert torch.equal(P.plain_embedding(table, [4, 0, 4]), F.embedding(torch.tensor([4, 0, 4]), table))


# --------------------------------------------------------------------------- whole model

def _model(tmp_path, which):
    folder, _ = make_model_folder(tmp_path, which)
    return P.read_model_folder(folder)


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_single_token_reduces_to_library_routines(tmp_path, which):
    """With one token the softmax is 1 and the rotation cancels out of the attention, so the whole
    model is a chain of library routines; this fixes where the norms stand, the residual sums, the
    order of the fused rows, the biases and which matrix the head reads."""
    cfg, w = _model(tmp_path, which)
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], P.plain_head_dim(cfg)
    H, eps = cfg["hidden_size"], cfg["rms_norm_eps"]
    tok = 5
    s = F.embedding(torch.tensor([tok]), w["model.embed_tokens.weight"])
    for i in range(cfg["num_hidden_layers"]):
        p = "model.layers.%d." % i
        h = F.rms_norm(s, (H,), w[p + "input_layernorm.weight"], eps)
        v = F.linear(h, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
        a = v.view(1, nkv, d).repeat_interleave(nh // nkv, dim=1).reshape(1, nh * d)
        s = s + F.linear(a, w[p + "self_attn.o_proj.weight"], w.get(p + "self_attn.o_proj.bias"))
        h = F.rms_norm(s, (H,), w[p + "post_attention_layernorm.weight"], eps)
        g = F.linear(h, w[p + "mlp.gate_proj.weight"], w.get(p + "mlp.gate_proj.bias"))
        u = F.linear(h, w[p + "mlp.up_proj.weight"], w.get(p + "mlp.up_proj.bias"))
        s = s + F.linear(F.silu(g) * u, w[p + "mlp.down_proj.weight"], w.get(p + "mlp.down_proj.bias"))
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    want = F.linear(F.rms_norm(s, (H,), w["model.norm.weight"], eps), head)
    got = P.plain_llama_forward(cfg, w, [tok])
    assert torch.allclose(got, want, atol=1e-5), (got - want).abs().max()
    # and at any position: one token attends to itself only
    assert torch.allclose(P.plain_llama_forward(cfg, w, [tok], start_position=17), want, atol=1e-5)


@pytest.mark.parametrize("which", ["A", "B"])
def test_shift_of_all_positions_changes_nothing(tmp_path, which):
    cfg, w = _model(tmp_path, which)
    toks = random_tokens(12, cfg["vocab_size"], 4)
    a = P.plain_llama_forward(cfg, w, toks)
    b = P.plain_llama_forward(cfg, w, toks, start_position=37)
    assert torch.allclose(a, b, atol=2e-4), (a - b).abs().max()


def test_positions_matter_and_the_model_is_causal(tmp_path):
    cfg, w = _model(tmp_path, "B")
    # random weights of std 0.02 make nearly flat attention; sharpen layer 0 so that order shows
    w = dict(w)
    w["model.layers.0.self_attn.q_proj.weight"] = w["model.layers.0.self_attn.q_proj.weight"] * 40
    w["model.layers.0.self_attn.k_proj.weight"] = w["model.layers.0.self_attn.k_proj.weight"] * 40
    toks = random_tokens(10, cfg["vocab_size"], 5)
    a = P.plain_llama_forward(cfg, w, toks)
    swapped = [toks[1], toks[0]] + toks[2:]
    b = P.plain_llama_forward(cfg, w, swapped)
    assert (a[-1] - b[-1]).abs().max() > 1e-4               # order of earlier tokens is seen through the rotation
    c = P.plain_llama_forward(cfg, w, toks[:6] + random_tokens(4, cfg["vocab_size"], 6))
    assert torch.equal(a[:6], c[:6])                        # later tokens are not


def test_schedule_and_window_options(tmp_path):
    cfg, w = _model(tmp_path, "A")
    toks = random_tokens(20, cfg["vocab_size"], 7)
    base = P.plain_llama_forward(cfg, w, toks)
    assert torch.equal(P.plain_llama_forward(cfg, w, toks, schedule=[(0, None), (1, None)]), base)
    twice = P.plain_llama_forward(cfg, w, toks, schedule=[(0, None), (1, None), (0, None)])
    assert not torch.allclose(twice, base, atol=1e-4)
    wide = P.plain_llama_forward(cfg, w, toks, windows={0: 64, 1: 64})
    assert torch.equal(wide, base)
    narrow = P.plain_llama_forward(cfg, w, toks, windows={0: 4})
    assert torch.allclose(narrow[:4], base[:4], atol=1e-6) and not torch.allclose(narrow[10:], base[10:], atol=1e-6)


def test_greedy_generate_is_argmax_of_forward(tmp_path):
    cfg, w = _model(tmp_path, "A")
    prompt = random_tokens(5, cfg["vocab_size"], 8)
    out = P.plain_greedy_generate(cfg, w, prompt, 3)
    ids = list(prompt)
    for t in out:
        assert t == int(P.plain_llama_forward(cfg, w, ids)[-1].argmax())
        ids.append(t)


# --------------------------------------------------------------------------- sampler maths

def test_penalties_by_hand():
    logits = torch.tensor([2.0, -1.0, 0.5, 3.0, -0.5])
    out = P.plain_apply_penalties(logits, prompt_ids=[0], output_ids=[1, 3, 3], presence=0.5, frequency=0.25,
                                  repetition=2.0)
    # 0: seen in prompt only: 2/2. 1: seen once in output: -1*2 - .25 - .5. 3: twice: 3/2 - .5 - .5. 2, 4 untouched
    assert torch.allclose(out, torch.tensor([1.0, -2.75, 0.5, 0.5, -0.5]))


def test_top_k_top_p_min_p():
    x = torch.log(torch.tensor([0.5, 0.25, 0.125, 0.0625, 0.0625]))
    keep = lambda y: set(torch.nonzero(torch.isfinite(y)).flatten().tolist())
    assert keep(P.plain_top_k_top_p(x, 2, 1.0)) == {0, 1}
    assert keep(P.plain_top_k_top_p(x, -1, 1.0)) == {0, 1, 2, 3, 4}
    assert keep(P.plain_top_k_top_p(x, -1, 0.7)) == {0, 1}          # mass of larger ones: 0, .5, .75 -> third is out
    assert keep(P.plain_top_k_top_p(x, -1, 0.01)) == {0}            # the largest always stays
    assert keep(P.plain_top_k_top_p(x, 3, 0.6)) == {0, 1}           # nucleus of the renormalised top 3
    assert keep(P.plain_min_p(x, 0.3)) == {0, 1}
    p = P.plain_sampling_distribution(x, temperature=0.5, top_k=3)
    want = torch.tensor([0.25, 0.0625, 0.015625, 0, 0])
    assert torch.allclose(p, want / want.sum(), atol=1e-6)


def test_the_noise_generator_is_philox4x32_10():
    """The counter-based generator behind the sampler's noise (tests/torch_ops.py, which the kernel's draws are
    compared with bit for bit on the GPU) against the algorithm's published known answers: the first output word
    for three (counter, key) pairs (all zeros; all ones; digits of pi). A wrong multiplier, key schedule, round
    count or word order fails all three."""
    import numpy as np
    from torch_ops import _philox_first

    def first(c, k):
        return int(_philox_first(np.array([c[0]], dtype=np.uint64), c[1], k[0], k[1], c[2], c[3])[0])

    assert first((0, 0, 0, 0), (0, 0)) == 0x6627E8D5
    assert first((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2) == 0x408F276D
    assert first((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0)) == 0xD16CFE09
