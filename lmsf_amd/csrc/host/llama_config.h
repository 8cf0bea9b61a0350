// The typed configuration of LlamaForCausalLM, read from config.json's own keys and validated.
//
// The reference parses config.json into a struct per architecture
// (core/src/model_executor/models/llama/config.rs:6-27, defaults :28-52) behind an accessor trait
// (core/src/model_executor/models/model.rs:8-37) and picks the struct by model_type
// (core/src/model_executor/models/model_factory.rs:268-333). This is that struct with the keys it lacks and a
// correct engine needs (head_dim, attention_bias, mlp_bias, rope_scaling, a list of end-of-sequence ids), with
// explicit defaults and one message per fault that names the key. Python's LlamaConfig is its face.
#pragma once
#include <cstdint>

extern "C" {

#define LMSF_MAX_EOS_IDS 16

typedef struct {
  int present;                    // 0: no rope_scaling (or rope_type "default")
  char rope_type[16];
  double factor, low_freq_factor, high_freq_factor;
  int64_t original_max_position_embeddings;
} LmsfRopeScaling;

typedef struct {
  int64_t vocab_size, max_position_embeddings, hidden_size, intermediate_size, num_hidden_layers, num_attention_heads,
      num_key_value_heads, head_dim;
  double rms_norm_eps, rope_theta;
  LmsfRopeScaling rope_scaling;
  int tie_word_embeddings, attention_bias, mlp_bias;
  char hidden_act[32], torch_dtype[16];
  int has_bos_token_id;
  int64_t bos_token_id;
  int n_eos_token_ids;
  int64_t eos_token_ids[LMSF_MAX_EOS_IDS];
} LmsfLlamaConfig;

// Both return 0, or 3 with the reason in lmsf_host_last_error().
int lmsf_llama_config_parse(const char* config_json, LmsfLlamaConfig* out);      // parses, fills defaults, validates
int lmsf_llama_config_validate(const LmsfLlamaConfig* config);
int lmsf_rope_scaling_parse(const char* rope_scaling_json, LmsfRopeScaling* out);   // the rope_scaling object alone
}
