"""Plain, slow implementation of the Llama forward pass and of the sampler's maths.

Whole sequences, no cache, no batching, float32 on the CPU; one function for each part.
It is written from the formulas of the reference (yinqiwen/lmsf, cited file:line below,
paths relative to the reference's root) and shares no code with the package under test:
it reads ``config.json`` as a plain dict and ``model.safetensors`` with the safetensors
package.

Where the reference has a quirk that a correct engine must not have (fixed rope base,
``sum + 1e-6`` in the decode softmax, logits at a padded column), the formula that the
text means is implemented and the quirk is named in the docstring.
"""
import json
import math
import os

import torch


# --------------------------------------------------------------------------- parts


def plain_embedding(table, token_ids):
    """x[t] = E[token[t]], a row gather without scale.

    core/src/model_executor/layers/vocab_parallel_embedding.rs:28-38 (index_select);
    core/src/model_executor/models/llama/llama.rs:413.
    """
    return table[torch.as_tensor(token_ids, dtype=torch.long)].to(torch.float32)


def plain_rms_norm(x, weight, eps):
    """y = x * rsqrt(mean(x^2) + eps) * w, all in float32.

    vllm/kernels/layernorm_kernels.cu:13-38 (variance = sum(x^2)/hidden, rsqrtf(var + eps),
    then times weight). No bias and no "+1" on the weight for Llama
    (core/src/model_executor/models/llama/llama.rs:362-374).
    """
    x = x.to(torch.float32)
    var = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight.to(torch.float32)


def plain_linear(x, weight, bias=None):
    """y = x W^T (+ b).

    core/src/model_executor/layers/linear.rs:44-106 (UnquantizedLinearWeights::apply:
    GEMM with the weight stored [out, in], then an optional broadcast add of the bias).
    """
    y = x.to(torch.float32) @ weight.to(torch.float32).t()
    if bias is not None:
        y = y + bias.to(torch.float32)
    return y


def plain_rope_inv_freq(rotary_dim, theta, scaling=None):
    """Inverse frequencies f_i = theta^(-2i/rotary_dim), i < rotary_dim/2, in float32.

    core/src/model_executor/layers/rotary_embedding.rs:46-58 (1 / base.powf(i / rotary_dim)
    for i in 0, 2, 4, ...). The reference fixes base to 10000 there (:105) although
    config.json's rope_theta is parsed (models/llama/config.rs:25-30); theta is used here.

    ``scaling`` is config.json's ``rope_scaling`` dict or None. For rope_type "llama3" each
    frequency is changed by its wavelength L = 2*pi/f: L < orig/high_freq_factor keeps f;
    L > orig/low_freq_factor gives f/factor; in between a linear blend
    (1-s) f/factor + s f with s = (orig/L - low) / (high - low). The reference has no
    rope_scaling; this is the published Llama-3.1 rule.
    """
    idx = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / torch.pow(torch.tensor(float(theta), dtype=torch.float32), idx / rotary_dim)
    if scaling is None:
        return inv_freq
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind in (None, "default"):
        return inv_freq
    if kind != "llama3":
        raise ValueError("plain implementation knows rope_type default and llama3 only")
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    out = []
    for f in inv_freq.tolist():
        wavelen = 2.0 * math.pi / f
        if wavelen < orig / high:
            out.append(f)
        elif wavelen > orig / low:
            out.append(f / factor)
        else:
            s = (orig / wavelen - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return torch.tensor(out, dtype=torch.float32)


def plain_rope_angles(positions, inv_freq):
    """angle[t, i] = position[t] * f_i as a float32 product.

    core/src/model_executor/layers/rotary_embedding.rs:58-66 (arange(max_pos) as f32,
    matmul with inv_freq, then cos and sin).
    """
    pos = torch.as_tensor(positions, dtype=torch.float32)
    return pos[:, None] * inv_freq[None, :].to(torch.float32)


def plain_apply_rope(x, positions, inv_freq, rotary_dim=None, neox=True):
    """Rotate the first ``rotary_dim`` components of every head of x [T, heads, d].

    NeoX style pairs (i, i + rot/2); GPT-J style pairs (2i, 2i+1):
    x' = x cos - y sin, y' = y cos + x sin
    (vllm/kernels/pos_encoding_kernels.cu:12-36). Llama uses NeoX style over the whole
    head (core/src/model_executor/models/llama/llama.rs:207-215: rotary_dim = head_dim,
    is_neox_style = true).
    """
    x = x.to(torch.float32)
    d = x.shape[-1]
    rot = d if rotary_dim is None else rotary_dim
    ang = plain_rope_angles(positions, inv_freq)  # [T, rot/2]
    cos = torch.cos(ang)[:, None, :]
    sin = torch.sin(ang)[:, None, :]
    out = x.clone()
    half = rot // 2
    if neox:
        a = x[..., :half]
        b = x[..., half:rot]
        out[..., :half] = a * cos - b * sin
        out[..., half:rot] = b * cos + a * sin
    else:
        a = x[..., 0:rot:2]
        b = x[..., 1:rot:2]
        out[..., 0:rot:2] = a * cos - b * sin
        out[..., 1:rot:2] = b * cos + a * sin
    return out


def plain_attention(q, k, v, scale=None, window=None):
    """Causal softmax attention of one sequence. q [T, nh, d]; k, v [T, nkv, d] -> [T, nh, d].

    core/src/model_executor/layers/attention.rs:91-103 (repeat_kv: kv head g serves query
    heads g*n_rep .. g*n_rep + n_rep - 1), :139-155 (float32; S = q k^T / sqrt(d); mask j > i
    with -inf; softmax over keys; P v). The decode kernel computes the same function for one
    query over the cached keys (vllm/kernels/attention/attention_kernels.cu:82-414) except
    that it divides by (sum + 1e-6) (:279), which is a quirk and is not reproduced.

    ``window`` = W keeps keys j with i - W < j <= i (the sliding window of
    core/src/sched/block_manager.rs:129-135 and core/src/worker/model_worker.rs:306-317).
    """
    q = q.to(torch.float32)
    k = k.to(torch.float32)
    v = v.to(torch.float32)
    T, nh, d = q.shape
    nkv = k.shape[1]
    n_rep = nh // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.empty(T, nh, v.shape[-1], dtype=torch.float32)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    dead = j > i
    if window is not None:
        dead = dead | (j <= i - window)
    for h in range(nh):
        g = h // n_rep
        s = (q[:, h, :] @ k[:, g, :].t()) * scale
        s = s.masked_fill(dead, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h, :] = p @ v[:, g, :]
    return out


def plain_silu(x):
    """silu(x) = x / (1 + exp(-x)). vllm/kernels/activation_kernels.cu:26-29."""
    return x / (1.0 + torch.exp(-x))


def plain_swiglu_mlp(x, w_gate, w_up, w_down, b_gate=None, b_up=None, b_down=None):
    """y = (silu(x Wg^T) * (x Wu^T)) Wd^T.

    core/src/model_executor/models/llama/llama.rs:234-248 (gate_up GEMM, silu_and_mul, down
    GEMM); vllm/kernels/activation_kernels.cu:31-42 (first half is the gate, second half
    is multiplied in).
    """
    g = plain_linear(x, w_gate, b_gate)
    u = plain_linear(x, w_up, b_up)
    return plain_linear(plain_silu(g) * u, w_down, b_down)


# --------------------------------------------------------------------------- whole model


def read_model_folder(folder):
    """(config dict, {tensor name: float32 tensor}) from config.json and model.safetensors."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    return cfg, {k: v.to(torch.float32) for k, v in tensors.items()}


def plain_head_dim(cfg):
    """Explicit head_dim key, else hidden/heads (core/src/common/config.rs:193-195)."""
    hd = cfg.get("head_dim")
    return int(hd) if hd else cfg["hidden_size"] // cfg["num_attention_heads"]


def plain_llama_layer(cfg, w, prefix, stream, positions, inv_freq, window=None, kv_from=None):
    """One pre-norm block on the residual stream [T, H]; returns (new stream, (k, v)).

    core/src/model_executor/models/llama/llama.rs:286-340: h1 = norm1(stream);
    stream += attn(h1); h2 = norm2(stream); stream += mlp(h2). The reference realises the
    additions inside the next fused add+norm (vllm/kernels/layernorm_kernels.cu:41-68);
    the sums are the same.

    ``kv_from`` = (k, v) of another layer: this layer then attends to those instead of its
    own keys and values (a layer that reads another layer's cache).
    """
    nh = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nh)
    d = plain_head_dim(cfg)
    eps = cfg["rms_norm_eps"]
    T = stream.shape[0]
    p = prefix
    h1 = plain_rms_norm(stream, w[p + ".input_layernorm.weight"], eps)
    q = plain_linear(h1, w[p + ".self_attn.q_proj.weight"], w.get(p + ".self_attn.q_proj.bias"))
    q = plain_apply_rope(q.view(T, nh, d), positions, inv_freq)
    if kv_from is None:
        k = plain_linear(h1, w[p + ".self_attn.k_proj.weight"], w.get(p + ".self_attn.k_proj.bias"))
        v = plain_linear(h1, w[p + ".self_attn.v_proj.weight"], w.get(p + ".self_attn.v_proj.bias"))
        k = plain_apply_rope(k.view(T, nkv, d), positions, inv_freq)
        v = v.view(T, nkv, d)
    else:
        k, v = kv_from
    a = plain_attention(q, k, v, scale=1.0 / math.sqrt(d), window=window)
    o = plain_linear(a.reshape(T, nh * d), w[p + ".self_attn.o_proj.weight"],
                     w.get(p + ".self_attn.o_proj.bias"))
    stream = stream + o
    h2 = plain_rms_norm(stream, w[p + ".post_attention_layernorm.weight"], eps)
    m = plain_swiglu_mlp(h2, w[p + ".mlp.gate_proj.weight"], w[p + ".mlp.up_proj.weight"],
                         w[p + ".mlp.down_proj.weight"], w.get(p + ".mlp.gate_proj.bias"),
                         w.get(p + ".mlp.up_proj.bias"), w.get(p + ".mlp.down_proj.bias"))
    return stream + m, (k, v)


def plain_llama_forward(cfg, w, token_ids, start_position=0, schedule=None, windows=None, last=None):
    """Logits [T, V] (float32) for every position of one whole sequence.

    core/src/model_executor/models/llama/llama.rs:397-476: embedding, the blocks in order,
    final norm, LM head. The reference takes the logits of the last padded column only
    (:466, a quirk for shorter prompts of a batch); here every position is returned.
    tie_word_embeddings true -> the head is the embedding table (the reference parses the
    key and ignores it, llama.rs:487-492).

    ``start_position`` shifts all positions (used by the shift invariance test).
    ``schedule`` is a list of (layer index, index of the earlier schedule entry whose keys and
    values are read, or None); default: every layer once, in order.
    ``windows`` maps a layer index to a sliding window length.
    ``last``: only the logits of the last ``last`` positions (the head is the costly part of a wide model).
    """
    d = plain_head_dim(cfg)
    inv_freq = plain_rope_inv_freq(d, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    T = len(token_ids)
    positions = list(range(start_position, start_position + T))
    stream = plain_embedding(w["model.embed_tokens.weight"], token_ids)
    if schedule is None:
        schedule = [(i, None) for i in range(cfg["num_hidden_layers"])]
    kvs = []
    for layer, src in schedule:
        window = None if windows is None else windows.get(layer)
        stream, kv = plain_llama_layer(cfg, w, "model.layers.%d" % layer, stream, positions,
                                       inv_freq, window=window,
                                       kv_from=None if src is None else kvs[src])
        kvs.append(kv)
    if last is not None:
        stream = stream[-last:]
    final = plain_rms_norm(stream, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return plain_linear(final, head)


def plain_greedy_generate(cfg, w, prompt, n_new):
    """Greedy continuation by re-running the whole sequence for every new token."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        logits = plain_llama_forward(cfg, w, ids)
        nxt = int(torch.argmax(logits[-1]).item())
        out.append(nxt)
        ids.append(nxt)
    return out


# --------------------------------------------------------------------------- sampler maths


def plain_apply_penalties(logits, prompt_ids, output_ids, presence, frequency, repetition):
    """Penalties on one row of logits [V], float32.

    core/src/model_executor/layers/sampler.rs:48-137: tokens seen in prompt or output get
    logits > 0 ? logits / r : logits * r; then logits -= frequency * count_in_output;
    then logits -= presence * [seen in output].
    """
    logits = logits.to(torch.float32).clone()
    V = logits.shape[0]
    out_counts = torch.zeros(V)
    for t in output_ids:
        out_counts[t] += 1
    seen = torch.zeros(V, dtype=torch.bool)
    for t in list(prompt_ids) + list(output_ids):
        seen[t] = True
    rep = torch.where(seen, torch.tensor(float(repetition)), torch.tensor(1.0))
    logits = torch.where(logits > 0, logits / rep, logits * rep)
    logits = logits - frequency * out_counts
    logits = logits - presence * (out_counts > 0).to(torch.float32)
    return logits


def plain_top_k_top_p(logits, top_k, top_p):
    """Mask one row of logits [V] with -inf outside top-k and the nucleus.

    core/src/model_executor/layers/sampler.rs:139-210: sort ascending; everything below the
    k-th largest value is masked; softmax of what is left; ascending cumulative sums <= 1 - p
    are masked; the largest is always kept; scattered back to vocabulary order.
    top_k <= 0 means the whole vocabulary.
    """
    logits = logits.to(torch.float32)
    V = logits.shape[0]
    k = V if top_k is None or top_k <= 0 else min(int(top_k), V)
    srt, idx = torch.sort(logits, descending=False, stable=True)
    kth = srt[V - k]
    srt = srt.masked_fill(srt < kth, float("-inf"))
    probs = torch.softmax(srt, dim=-1)
    csum = torch.cumsum(probs, dim=-1)
    mask = csum <= (1.0 - float(top_p))
    mask[-1] = False
    srt = srt.masked_fill(mask, float("-inf"))
    out = torch.empty_like(srt)
    out[idx] = srt
    return out


def plain_min_p(logits, min_p):
    """Mask tokens whose probability is below min_p * max probability.

    core/src/model_executor/layers/sampler.rs:305-325.
    """
    probs = torch.softmax(logits.to(torch.float32), dim=-1)
    return logits.masked_fill(probs < float(min_p) * probs.max(), float("-inf"))


def plain_sampling_distribution(logits, temperature=1.0, top_k=-1, top_p=1.0, min_p=0.0,
                                prompt_ids=(), output_ids=(), presence=0.0, frequency=0.0,
                                repetition=1.0):
    """The categorical distribution the sampler draws from, for one row.

    Order of core/src/model_executor/layers/sampler.rs:839-922: penalties, divide by the
    temperature, top-k/top-p, min-p, float32 softmax. (The reference applies the first two
    in the model's dtype, a quirk; float32 here.)
    """
    x = logits.to(torch.float32)
    if presence != 0.0 or frequency != 0.0 or repetition != 1.0:
        x = plain_apply_penalties(x, prompt_ids, output_ids, presence, frequency, repetition)
    x = x / float(temperature)
    if (top_k is not None and top_k > 0) or top_p < 1.0:
        x = plain_top_k_top_p(x, top_k, top_p)
    if min_p > 0.0:
        x = plain_min_p(x, min_p)
    return torch.softmax(x, dim=-1)
