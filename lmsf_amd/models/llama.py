"""LlamaForCausalLM as a ModelSpec: which parts, with which parameters, under which names.

Dense decoder with grouped-query attention, rotary embedding (NeoX pairing over the whole head),
RMSNorm and a SiLU-gated feed-forward (core/src/model_executor/models/llama/llama.rs:45-536).
Checkpoint names: model.embed_tokens.weight, model.layers.{i}.{input_layernorm,
post_attention_layernorm}.weight, model.layers.{i}.self_attn.{q,k,v,o}_proj.weight,
model.layers.{i}.mlp.{gate,up,down}_proj.weight, model.norm.weight, lm_head.weight
(llama.rs:185-189, :265-267, :353-373, :485-495), plus the optional biases.
"""
from ..config.model_config import LlamaConfig
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    position = PartSpec("rotary", {
        "head_dim": cfg.head_dim,
        "theta": cfg.rope_theta,
        "scaling": None if cfg.rope_scaling is None else cfg.rope_scaling.to_dict(),
        "style": "neox",
    })
    mixer = PartSpec("paged_attention", {
        "prefix": "self_attn",
        "hidden_size": cfg.hidden_size,
        "num_heads": cfg.num_attention_heads,
        "num_kv_heads": cfg.num_key_value_heads,
        "head_dim": cfg.head_dim,
        "position": position,
        "qkv_bias": cfg.attention_bias,
        "out_bias": cfg.attention_bias,
    })
    ffn = PartSpec("gated_mlp", {
        "prefix": "mlp",
        "hidden_size": cfg.hidden_size,
        "intermediate_size": cfg.intermediate_size,
        "activation": cfg.hidden_act,
        "bias": cfg.mlp_bias,
    })

    def norm(prefix):
        return PartSpec("rms_norm", {"prefix": prefix, "size": cfg.hidden_size, "eps": cfg.rms_norm_eps})

    layers = tuple(
        LayerSpec(prefix="model.layers.%d" % i, block=PartSpec("prenorm_residual"), mixer=mixer, feed_forward=ffn,
                  norms={"input": norm("input_layernorm"), "post_mixer": norm("post_attention_layernorm")})
        for i in range(cfg.num_hidden_layers))
    head_weight = "model.embed_tokens.weight" if cfg.tie_word_embeddings else "lm_head.weight"
    return ModelSpec(
        embedding=PartSpec("token_embedding", {"prefix": "model.embed_tokens", "vocab_size": cfg.vocab_size,
                                               "hidden_size": cfg.hidden_size}),
        layers=layers,
        schedule=tuple(ScheduleEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=norm("model.norm"),
        head=PartSpec("lm_head", {"prefix": "lm_head", "vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                  "weight_name": head_weight}),
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
    )


# checkpoints of tied models often still carry lm_head.weight; rotary buffers of old exports are ignored too
LLAMA_TOLERATED = ("lm_head.weight", ".rotary_emb.inv_freq")

register_architecture("LlamaForCausalLM", "llama", LlamaConfig, build_llama_spec, tolerated_tensors=LLAMA_TOLERATED)
