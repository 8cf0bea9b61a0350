#include "llama_config.h"

#include <cmath>
#include <cstring>
#include <string>

#include "cache_manager.h"   // Error, fail
#include "json.h"

namespace lmsf {
namespace {

const Json* member(const Json& d, const char* key) {
  const Json* v = d.find(key);
  return (v == nullptr || v->kind == Json::kNull) ? nullptr : v;     // null counts as absent
}

[[noreturn]] void wrong_type(const char* key, const Json& v, const char* expected) {
  fail(kValueError, "config.json: key '%s' has value %s, expected %s", key, v.repr().c_str(), expected);
}
[[noreturn]] void missing(const char* key) { fail(kValueError, "config.json: required key '%s' is missing", key); }

bool take_int(const Json& d, const char* key, int64_t* out) {
  const Json* v = member(d, key);
  if (v == nullptr) return false;
  if (v->kind != Json::kNumber || v->number != std::floor(v->number) || std::fabs(v->number) > 9e15)
    wrong_type(key, *v, "int");
  *out = (int64_t)v->number;
  return true;
}
int64_t need_int(const Json& d, const char* key) {
  int64_t v = 0;
  if (!take_int(d, key, &v)) missing(key);
  return v;
}
bool take_float(const Json& d, const char* key, double* out) {
  const Json* v = member(d, key);
  if (v == nullptr) return false;
  if (v->kind != Json::kNumber) wrong_type(key, *v, "float");
  *out = v->number;
  return true;
}
double need_float(const Json& d, const char* key) {
  double v = 0;
  if (!take_float(d, key, &v)) missing(key);
  return v;
}
bool take_bool(const Json& d, const char* key, bool fallback) {
  const Json* v = member(d, key);
  if (v == nullptr) return fallback;
  if (v->kind != Json::kBool) wrong_type(key, *v, "bool");
  return v->boolean;
}
std::string take_str(const Json& d, const char* key, const char* fallback) {
  const Json* v = member(d, key);
  if (v == nullptr) return fallback;
  if (v->kind != Json::kString) wrong_type(key, *v, "str");
  return v->text;
}
void put(char* dst, size_t cap, const std::string& s, const char* key) {
  if (s.size() + 1 > cap) fail(kValueError, "config.json: key '%s' has value '%s', which is too long", key, s.c_str());
  std::memcpy(dst, s.c_str(), s.size() + 1);
}

void parse_rope_scaling(const Json* v, LmsfRopeScaling* out) {
  std::memset(out, 0, sizeof(*out));
  if (v == nullptr || v->kind == Json::kNull) return;
  if (v->kind != Json::kObject)
    fail(kValueError, "config.json: 'rope_scaling' must be an object or null, got %s", v->repr().c_str());
  const Json* kind = member(*v, "rope_type");
  if (kind == nullptr) kind = member(*v, "type");
  const std::string name = kind == nullptr ? "default" : kind->kind == Json::kString ? kind->text : kind->repr();
  if (name != "default" && name != "llama3")
    fail(kValueError, "config.json: rope_scaling.rope_type '%s' is not supported (known: default, llama3)", name.c_str());
  if (name == "default") return;
  out->present = 1;
  put(out->rope_type, sizeof(out->rope_type), name, "rope_scaling.rope_type");
  out->factor = need_float(*v, "factor");
  out->low_freq_factor = need_float(*v, "low_freq_factor");
  out->high_freq_factor = need_float(*v, "high_freq_factor");
  out->original_max_position_embeddings = need_int(*v, "original_max_position_embeddings");
  if (out->factor <= 0 || out->original_max_position_embeddings <= 0)
    fail(kValueError, "config.json: rope_scaling factor and original_max_position_embeddings must be > 0");
  if (out->high_freq_factor <= out->low_freq_factor)
    fail(kValueError, "config.json: rope_scaling.high_freq_factor must exceed low_freq_factor");
}

void validate(const LmsfLlamaConfig& c) {
  const struct {
    const char* name;
    int64_t value;
  } positive[] = {{"vocab_size", c.vocab_size},
                  {"hidden_size", c.hidden_size},
                  {"intermediate_size", c.intermediate_size},
                  {"num_hidden_layers", c.num_hidden_layers},
                  {"num_attention_heads", c.num_attention_heads},
                  {"num_key_value_heads", c.num_key_value_heads},
                  {"head_dim", c.head_dim},
                  {"max_position_embeddings", c.max_position_embeddings}};
  for (const auto& p : positive)
    if (p.value <= 0) fail(kValueError, "config.json: %s must be > 0, got %lld", p.name, (long long)p.value);
  if (c.num_attention_heads % c.num_key_value_heads != 0)
    fail(kValueError, "config.json: num_attention_heads %lld is not a multiple of num_key_value_heads %lld",
         (long long)c.num_attention_heads, (long long)c.num_key_value_heads);
  if (c.head_dim % 2 != 0)
    fail(kValueError, "config.json: head_dim %lld must be even for rotary embedding", (long long)c.head_dim);
  if (!(c.rms_norm_eps > 0)) fail(kValueError, "config.json: rms_norm_eps must be > 0");
  if (!(c.rope_theta > 0)) fail(kValueError, "config.json: rope_theta must be > 0");
  if (std::strcmp(c.hidden_act, "silu") != 0)
    fail(kValueError, "config.json: hidden_act '%s' is not supported by LlamaForCausalLM (silu)", c.hidden_act);
  bool known = false;
  for (const char* t : {"float32", "bfloat16", "float16", "half", "float"}) known = known || std::strcmp(c.torch_dtype, t) == 0;
  if (!known)
    fail(kValueError, "config.json: torch_dtype '%s' is not one of float32, bfloat16, float16, half, float", c.torch_dtype);
  if (c.n_eos_token_ids < 0 || c.n_eos_token_ids > LMSF_MAX_EOS_IDS)
    fail(kValueError, "config.json: eos_token_id lists %d ids, at most %d are taken", c.n_eos_token_ids, LMSF_MAX_EOS_IDS);
  for (int i = 0; i < c.n_eos_token_ids; ++i)
    if (c.eos_token_ids[i] < 0 || c.eos_token_ids[i] >= c.vocab_size)
      fail(kValueError, "config.json: eos_token_id %lld outside vocabulary of %lld", (long long)c.eos_token_ids[i],
           (long long)c.vocab_size);
  if (c.rope_scaling.present) {
    if (c.rope_scaling.factor <= 0 || c.rope_scaling.original_max_position_embeddings <= 0)
      fail(kValueError, "config.json: rope_scaling factor and original_max_position_embeddings must be > 0");
    if (c.rope_scaling.high_freq_factor <= c.rope_scaling.low_freq_factor)
      fail(kValueError, "config.json: rope_scaling.high_freq_factor must exceed low_freq_factor");
  }
}

void parse(const std::string& text, LmsfLlamaConfig* out) {
  const Json d = parse_json(text);
  if (d.kind != Json::kObject) fail(kValueError, "config.json does not hold a JSON object");
  LmsfLlamaConfig c;
  std::memset(&c, 0, sizeof(c));
  c.hidden_size = need_int(d, "hidden_size");
  c.num_attention_heads = need_int(d, "num_attention_heads");
  if (c.num_attention_heads <= 0) fail(kValueError, "config.json: num_attention_heads must be > 0");
  if (!take_int(d, "head_dim", &c.head_dim)) {
    if (c.hidden_size % c.num_attention_heads != 0)
      fail(kValueError, "config.json: hidden_size %lld is not a multiple of num_attention_heads %lld and no head_dim is given",
           (long long)c.hidden_size, (long long)c.num_attention_heads);
    c.head_dim = c.hidden_size / c.num_attention_heads;
  }
  const Json* eos = member(d, "eos_token_id");
  if (eos != nullptr) {
    Json wrapped;
    const Json* list = eos;
    if (eos->kind != Json::kArray) {
      wrapped.kind = Json::kArray;
      wrapped.items.push_back(*eos);
      list = &wrapped;
    }
    if (list->items.size() > LMSF_MAX_EOS_IDS)
      fail(kValueError, "config.json: eos_token_id lists %zu ids, at most %d are taken", list->items.size(), LMSF_MAX_EOS_IDS);
    for (const Json& e : list->items) {
      if (e.kind != Json::kNumber || e.number != std::floor(e.number)) wrong_type("eos_token_id", *eos, "int or list of int");
      c.eos_token_ids[c.n_eos_token_ids++] = (int64_t)e.number;
    }
  }
  // torch_dtype, else dtype, else bfloat16
  put(c.torch_dtype, sizeof(c.torch_dtype), take_str(d, "torch_dtype", take_str(d, "dtype", "bfloat16").c_str()), "torch_dtype");
  c.vocab_size = need_int(d, "vocab_size");
  c.max_position_embeddings = need_int(d, "max_position_embeddings");
  c.has_bos_token_id = take_int(d, "bos_token_id", &c.bos_token_id) ? 1 : 0;
  c.intermediate_size = need_int(d, "intermediate_size");
  c.num_hidden_layers = need_int(d, "num_hidden_layers");
  if (!take_int(d, "num_key_value_heads", &c.num_key_value_heads))
    c.num_key_value_heads = c.num_attention_heads;                    // core/src/model_executor/models/model.rs:24-26
  c.rms_norm_eps = need_float(d, "rms_norm_eps");
  if (!take_float(d, "rope_theta", &c.rope_theta)) c.rope_theta = 10000.0;   // llama/config.rs:28-30
  parse_rope_scaling(d.find("rope_scaling"), &c.rope_scaling);
  c.tie_word_embeddings = take_bool(d, "tie_word_embeddings", false) ? 1 : 0;
  c.attention_bias = take_bool(d, "attention_bias", false) ? 1 : 0;
  c.mlp_bias = take_bool(d, "mlp_bias", false) ? 1 : 0;
  put(c.hidden_act, sizeof(c.hidden_act), take_str(d, "hidden_act", "silu"), "hidden_act");
  validate(c);
  *out = c;
}

}  // namespace

void llama_config_parse(const std::string& text, LmsfLlamaConfig* out) { parse(text, out); }
void llama_config_validate(const LmsfLlamaConfig& c) { validate(c); }
void rope_scaling_parse(const std::string& text, LmsfRopeScaling* out) {
  const Json v = parse_json(text);
  parse_rope_scaling(&v, out);
}

}  // namespace lmsf
