// Drives the C API of the host library (cache manager, scheduler, step metadata) the way the engine does,
// over a random workload that reaches admission, portions, decoding, preemption, refusal, capping, abort and
// the error paths. Built with -fsanitize=address,undefined by tests/test_host_sanitizers.py: what it checks is
// what the sanitizers and the library's own check_invariants find. Test code only.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <string>
#include <vector>

#include <unistd.h>

#include "llama_config.h"

extern "C" {
typedef struct {
  const char* name;
  char dtype[8];
  int ndim;
  int64_t shape[8];
  int64_t begin, end;
} LmsfTensorRecord;
int lmsf_safetensors_open(const char* path, void** out);
void lmsf_safetensors_close(void* file);
int64_t lmsf_safetensors_count(void* file);
int lmsf_safetensors_record(void* file, int64_t index, LmsfTensorRecord* out);
const void* lmsf_safetensors_data(void* file, int64_t* size);
int lmsf_host_abi_version();
const char* lmsf_host_last_error();
int lmsf_pool_create(int num_pages, void** out);
void lmsf_pool_destroy(void* pool);
int lmsf_pool_num_free(void* pool);
int lmsf_pool_allocate(void* pool, int* page);
int lmsf_pool_release(void* pool, int page);
int lmsf_cm_create(int n_groups, const int* page_size, const int* num_pages, const int* window, int num_state_slots,
                   void** out);
void lmsf_cm_destroy(void* cm);
int lmsf_cm_has_request(void* cm, int64_t rid);
int lmsf_cm_num_free_state_slots(void* cm);
int lmsf_cm_num_free_pages(void* cm, int group, int* out);
int lmsf_cm_request_info(void* cm, int64_t rid, int64_t* info);
int lmsf_cm_block_table(void* cm, int64_t rid, int group, int* out, int cap, int* len, int* first_live);
int lmsf_cm_live_requests(void* cm, int64_t* out, int cap, int* count);
int lmsf_cm_append(void* cm, int64_t rid, int64_t n_new, int64_t* start);
int lmsf_cm_free_request(void* cm, int64_t rid);
int lmsf_cm_slot_mapping(void* cm, int64_t rid, int group, int64_t start, int64_t n, int* out);
int lmsf_cm_check_invariants(void* cm);
int lmsf_cm_begin_step(void* cm, int S, const int64_t* rids, const int* lens, int64_t* starts, unsigned char* added);
int lmsf_cm_abort_step(void* cm, int S, const int64_t* rids, const unsigned char* added);
int lmsf_cm_commit_step(void* cm, int S, const int64_t* rids);
int lmsf_cm_step_widths(void* cm, int S, const int64_t* rids, int* widths);
int lmsf_step_layout(int64_t N, int64_t S, int64_t R, int G, const int* widths, int64_t* offsets, int64_t* total);
int lmsf_cm_fill_step(void* cm, int S, const int64_t* rids, const int64_t* starts, const int* lens, const int* widths,
                      const int64_t* offsets, int32_t* buffer);
int lmsf_sched_create(void* cm, int64_t max_num_batched_tokens, int max_num_seqs, int64_t max_model_len,
                      int64_t prefill_chunk_size, double watermark, void** out);
void lmsf_sched_destroy(void* s);
int lmsf_sched_add(void* s, int64_t id, int64_t arrival, int64_t length);
int lmsf_sched_set_progress(void* s, int n, const int64_t* ids, const int64_t* lengths, const int64_t* computed);
int lmsf_sched_abort(void* s, int64_t id, int* found);
int lmsf_sched_finish(void* s, int64_t id);
int lmsf_sched_schedule(void* s, int* counts);
int lmsf_sched_plan(void* s, int64_t* ids, int64_t* starts, int64_t* n_tokens, int* samples, int64_t* preempted,
                    int64_t* ignored, int64_t* capped);
int lmsf_sched_queue(void* s, int which, int64_t* out, int cap, int* count);
int64_t lmsf_sched_num_preemptions(void* s);
}

#define MUST(call)                                                                              \
  do {                                                                                          \
    int rc_ = (call);                                                                           \
    if (rc_ != 0) {                                                                             \
      std::fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, rc_, lmsf_host_last_error()); \
      return 1;                                                                                 \
    }                                                                                           \
  } while (0)
#define MUST_FAIL(call, want)                                                                   \
  do {                                                                                          \
    int rc_ = (call);                                                                           \
    if (rc_ != (want)) {                                                                        \
      std::fprintf(stderr, "%s:%d: %s -> %d, expected %d\n", __FILE__, __LINE__, #call, rc_, (want)); \
      return 1;                                                                                 \
    }                                                                                           \
  } while (0)

struct Seq {
  int64_t length, computed, target;   // target: the length at which the driver finishes it
};

static uint64_t rng_state = 12345;
static uint32_t rnd(uint32_t n) {
  rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
  return (uint32_t)(rng_state >> 33) % n;
}

int main(int argc, char** argv) {
  if (argc > 1) rng_state = std::strtoull(argv[1], nullptr, 10);
  if (lmsf_host_abi_version() < 1) return 1;

  // the configuration reader: good text, every kind of broken text, and random cuts and flips of good text
  {
    const std::string good =
        "{\"architectures\": [\"LlamaForCausalLM\"], \"hidden_size\": 64, \"num_attention_heads\": 4, "
        "\"num_key_value_heads\": 2, \"intermediate_size\": 176, \"num_hidden_layers\": 2, \"vocab_size\": 256, "
        "\"max_position_embeddings\": 128, \"rms_norm_eps\": 1e-5, \"rope_theta\": 10000.0, \"eos_token_id\": [2, 3], "
        "\"tie_word_embeddings\": true, \"hidden_act\": \"si\\u006cu\", \"torch_dtype\": \"bfloat16\", "
        "\"rope_scaling\": {\"rope_type\": \"llama3\", \"factor\": 8.0, \"low_freq_factor\": 1.0, "
        "\"high_freq_factor\": 4.0, \"original_max_position_embeddings\": 64}}";
    LmsfLlamaConfig cfg;
    MUST(lmsf_llama_config_parse(good.c_str(), &cfg));
    if (cfg.head_dim != 16 || cfg.n_eos_token_ids != 2 || !cfg.rope_scaling.present || std::string(cfg.hidden_act) != "silu")
      return 1;
    MUST(lmsf_llama_config_validate(&cfg));
    cfg.head_dim = 15;
    MUST_FAIL(lmsf_llama_config_validate(&cfg), 3);
    for (const char* bad : {"", "{", "[1, 2", "{\"a\": }", "{\"hidden_size\": 1e999}", "\"text\"", "{\"a\": \"\\u12\"}",
                            "{\"hidden_size\": 64} trailing", "nul", "{\"a\" 1}"})
      MUST_FAIL(lmsf_llama_config_parse(bad, &cfg), 3);
    std::string deep(200, '[');
    MUST_FAIL(lmsf_llama_config_parse(deep.c_str(), &cfg), 3);
    for (int it = 0; it < 400; ++it) {
      std::string t = good;
      if (rnd(2)) t.resize(rnd((uint32_t)t.size()));
      for (int k = (int)rnd(4); k > 0 && !t.empty(); --k) t[rnd((uint32_t)t.size())] = (char)(32 + rnd(95));
      const int rc = lmsf_llama_config_parse(t.c_str(), &cfg);
      if (rc != 0 && rc != 3) return 1;
    }
    LmsfRopeScaling rs;
    MUST(lmsf_rope_scaling_parse("{\"type\": \"default\"}", &rs));
    if (rs.present) return 1;
    MUST_FAIL(lmsf_rope_scaling_parse("{\"rope_type\": \"yarn\"}", &rs), 3);
  }

  // the checkpoint reader: a good file, then cuts and flips of its header and a shortened data section; whatever it
  // accepts is read to the last byte of every tensor (the sanitizer sees a read outside the mapping)
  {
    const std::string good =
        "{\"__metadata__\": {\"format\": \"pt\"}, \"b\": {\"dtype\": \"BF16\", \"shape\": [3, 4], \"data_offsets\": [16, 40]}, "
        "\"a\": {\"dtype\": \"F32\", \"shape\": [2, 2], \"data_offsets\": [0, 16]}, "
        "\"e\": {\"dtype\": \"I32\", \"shape\": [0], \"data_offsets\": [40, 40]}}";
    char path[] = "/tmp/lmsf_san_XXXXXX";
    const int fd = mkstemp(path);
    if (fd < 0) return 1;
    close(fd);
    const auto write_file = [&](const std::string& header, size_t data_bytes, uint64_t claimed) {
      FILE* f = std::fopen(path, "wb");
      if (!f) std::exit(1);
      unsigned char len[8];
      for (int i = 0; i < 8; ++i) len[i] = (unsigned char)(claimed >> (8 * i));
      std::fwrite(len, 1, 8, f);
      std::fwrite(header.data(), 1, header.size(), f);
      for (size_t i = 0; i < data_bytes; ++i) std::fputc((int)(i & 0xff), f);
      std::fclose(f);
    };
    const auto open_and_read = [&](long* sum) {
      void* file = nullptr;
      const int rc = lmsf_safetensors_open(path, &file);
      if (rc != 0) return rc;
      int64_t size = 0;
      const unsigned char* data = (const unsigned char*)lmsf_safetensors_data(file, &size);
      for (int64_t i = 0; i < lmsf_safetensors_count(file); ++i) {
        LmsfTensorRecord r;
        if (lmsf_safetensors_record(file, i, &r) != 0) continue;
        if (r.begin < 0 || r.end > size || r.begin > r.end) std::exit(1);
        for (int64_t b = r.begin; b < r.end; ++b) *sum += data[b];
      }
      lmsf_safetensors_close(file);
      return 0;
    };
    long sum = 0;
    write_file(good, 40, good.size());
    MUST(open_and_read(&sum));
    if (sum != 40 * 39 / 2) return 1;
    write_file(good, 39, good.size());                   // a byte short
    MUST_FAIL(open_and_read(&sum), 3);
    write_file(good, 40, (uint64_t)1 << 40);             // a header longer than the file
    MUST_FAIL(open_and_read(&sum), 3);
    write_file(good, 0, 0);
    MUST_FAIL(open_and_read(&sum), 3);
    for (const char* bad :
         {"{\"a\": {\"dtype\": \"F32\", \"shape\": [2, 2], \"data_offsets\": [0, 12]}}",          // bytes against shape
          "{\"a\": {\"dtype\": \"F8\", \"shape\": [4], \"data_offsets\": [0, 4]}}",              // unknown dtype
          "{\"a\": {\"dtype\": \"U8\", \"shape\": [8], \"data_offsets\": [0, 8]}, "
          "\"b\": {\"dtype\": \"U8\", \"shape\": [8], \"data_offsets\": [4, 12]}}",               // overlap
          "{\"a\": {\"dtype\": \"U8\", \"shape\": [4], \"data_offsets\": [0, 4]}, "
          "\"a\": {\"dtype\": \"U8\", \"shape\": [4], \"data_offsets\": [4, 8]}}",                // one name twice
          "{\"a\": {\"dtype\": \"U8\", \"shape\": [-4], \"data_offsets\": [0, 4]}}",
          "{\"a\": {\"dtype\": \"U8\", \"shape\": [4.0], \"data_offsets\": [0, 4]}}",
          "{\"a\": {\"dtype\": \"I64\", \"shape\": [4294967296, 4294967296], \"data_offsets\": [0, 0]}}",
          "{\"a\": [1, 2]}", "[]", "{\"a\": {\"dtype\": \"U8\", \"shape\": [4]}}"}) {
      write_file(bad, 40, std::string(bad).size());
      MUST_FAIL(open_and_read(&sum), 3);
    }
    for (int it = 0; it < 300; ++it) {
      std::string t = good;
      if (rnd(3) == 0) t.resize(rnd((uint32_t)t.size()));
      for (int k = (int)rnd(4); k > 0 && !t.empty(); --k) t[rnd((uint32_t)t.size())] = (char)(32 + rnd(95));
      write_file(t, rnd(48), rnd(8) ? t.size() : rnd(200));
      const int rc = open_and_read(&sum);
      if (rc != 0 && rc != 3) return 1;
    }
    unlink(path);
    void* none = nullptr;
    MUST_FAIL(lmsf_safetensors_open(path, &none), 3);   // no such file
  }

  // the pool alone, with its error paths
  void* pool = nullptr;
  MUST(lmsf_pool_create(3, &pool));
  int page = -1, p2 = -1, p3 = -1;
  MUST(lmsf_pool_allocate(pool, &page));
  MUST(lmsf_pool_allocate(pool, &p2));
  MUST(lmsf_pool_allocate(pool, &p3));
  MUST_FAIL(lmsf_pool_allocate(pool, &p3), 2);     // out of pages
  MUST(lmsf_pool_release(pool, p2));
  MUST_FAIL(lmsf_pool_release(pool, p2), 1);       // freed twice
  MUST_FAIL(lmsf_pool_release(pool, 99), 1);       // never held
  if (lmsf_pool_num_free(pool) != 1) return 1;
  lmsf_pool_destroy(pool);

  // two groups: all keys in pages of 8, a window of 24 keys in pages of 16; few pages, few slots
  const int page_size[2] = {8, 16}, num_pages[2] = {20, 12}, window[2] = {0, 24};   // 160 tokens: fewer than the model allows
  void* cm = nullptr;
  MUST(lmsf_cm_create(2, page_size, num_pages, window, 6, &cm));
  void* sched = nullptr;
  MUST(lmsf_sched_create(cm, 48, 5, 200, 16, 0.01, &sched));

  int64_t start = 0, info[8] = {0};
  MUST_FAIL(lmsf_cm_append(cm, 777, 3, &start), 1);          // unknown request
  MUST_FAIL(lmsf_cm_free_request(cm, 777), 1);
  MUST_FAIL(lmsf_cm_request_info(cm, 777, info), 1);

  std::map<int64_t, Seq> live;
  int64_t next_id = 1, arrival = 0, steps = 0, finished = 0, ignored_n = 0, capped_n = 0, aborted = 0;
  std::vector<int32_t> buffer;
  for (int it = 0; it < 600 || !live.empty(); ++it) {
    if (it < 600 && rnd(3) == 0) {
      const int64_t id = next_id++;
      int64_t len = 1 + rnd(60);
      if (rnd(20) == 0) len = 120 + rnd(100);      // some too long for the model or for the pool, some that outgrow the pool
      MUST(lmsf_sched_add(sched, id, arrival++, len));
      live[id] = Seq{len, 0, len + 1 + (int64_t)rnd(40)};
    }
    if (!live.empty() && rnd(25) == 0) {           // abort a request, wherever it is
      auto pick = live.begin();
      std::advance(pick, rnd((uint32_t)live.size()));
      int found = 0;
      MUST(lmsf_sched_abort(sched, pick->first, &found));
      if (!found) return 1;
      live.erase(pick);
      ++aborted;
    }
    if (live.empty()) continue;
    std::vector<int64_t> ids, lens, comp;
    for (auto& kv : live) {
      ids.push_back(kv.first);
      lens.push_back(kv.second.length);
      comp.push_back(kv.second.computed);
    }
    MUST(lmsf_sched_set_progress(sched, (int)ids.size(), ids.data(), lens.data(), comp.data()));
    int counts[4] = {0, 0, 0, 0};
    MUST(lmsf_sched_schedule(sched, counts));
    const int ns = counts[0];
    std::vector<int64_t> sid(ns + 1), sstart(ns + 1), stok(ns + 1), pre(counts[1] + 1), ign(counts[2] + 1), cap(counts[3] + 1);
    std::vector<int> samples(ns + 1);
    MUST(lmsf_sched_plan(sched, sid.data(), sstart.data(), stok.data(), samples.data(), pre.data(), ign.data(), cap.data()));
    for (int i = 0; i < counts[1]; ++i) live[pre[i]].computed = 0;
    for (int i = 0; i < counts[2]; ++i) { live.erase(ign[i]); ++ignored_n; }
    for (int i = 0; i < counts[3]; ++i) { live.erase(cap[i]); ++capped_n; }
    if (ns == 0) {
      MUST(lmsf_cm_check_invariants(cm));
      continue;
    }
    // the executor's part: take the pages, write the step's metadata, commit
    std::vector<int> n_new(ns);
    int64_t N = 0, R = 0;
    for (int i = 0; i < ns; ++i) {
      n_new[i] = (int)stok[i];
      N += stok[i];
      R += samples[i];
      if (sstart[i] != live[sid[i]].computed) {
        std::fprintf(stderr, "request %ld planned from %ld but has %ld computed\n", (long)sid[i], (long)sstart[i],
                     (long)live[sid[i]].computed);
        return 1;
      }
    }
    if (N > 48) return 1;                            // the token budget
    std::vector<int64_t> starts(ns);
    std::vector<unsigned char> added(ns);
    MUST(lmsf_cm_begin_step(cm, ns, sid.data(), n_new.data(), starts.data(), added.data()));
    if (rnd(15) == 0) {                              // a step that fails after it took its pages
      MUST(lmsf_cm_abort_step(cm, ns, sid.data(), added.data()));
      MUST(lmsf_cm_check_invariants(cm));
      continue;
    }
    int widths[2] = {0, 0};
    MUST(lmsf_cm_step_widths(cm, ns, sid.data(), widths));
    int64_t offsets[32] = {0}, total = 0;
    MUST(lmsf_step_layout(N, ns, R, 2, widths, offsets, &total));
    buffer.assign((size_t)total, -7);
    MUST(lmsf_cm_fill_step(cm, ns, sid.data(), starts.data(), n_new.data(), widths, offsets, buffer.data()));
    std::vector<int> slots((size_t)stok[0]);
    MUST(lmsf_cm_slot_mapping(cm, sid[0], 0, starts[0], stok[0], slots.data()));
    for (int s : slots)
      if (s < 0 || s >= 20 * 8) return 1;
    int table[64], len = 0, first_live = 0;
    MUST(lmsf_cm_block_table(cm, sid[0], 1, table, 64, &len, &first_live));
    MUST(lmsf_cm_commit_step(cm, ns, sid.data()));
    ++steps;
    for (int i = 0; i < ns; ++i) {
      Seq& s = live[sid[i]];
      s.computed += stok[i];
      if (samples[i]) {
        s.length += 1;
        if (s.length >= s.target || s.length >= 200) {
          MUST(lmsf_sched_finish(sched, sid[i]));
          live.erase(sid[i]);
          ++finished;
        }
      }
    }
    MUST(lmsf_cm_check_invariants(cm));
    if (it > 100000) {
      std::fprintf(stderr, "the workload does not drain\n");
      return 1;
    }
  }
  int free0 = 0, free1 = 0, count = 0;
  MUST(lmsf_cm_num_free_pages(cm, 0, &free0));
  MUST(lmsf_cm_num_free_pages(cm, 1, &free1));
  MUST(lmsf_cm_live_requests(cm, nullptr, 0, &count));
  if (free0 != 20 || free1 != 12 || count != 0 || lmsf_cm_num_free_state_slots(cm) != 6) {
    std::fprintf(stderr, "left over: %d %d pages free, %d requests\n", free0, free1, count);
    return 1;
  }
  std::printf("OK steps=%ld finished=%ld ignored=%ld capped=%ld aborted=%ld preemptions=%ld\n", (long)steps,
              (long)finished, (long)ignored_n, (long)capped_n, (long)aborted, (long)lmsf_sched_num_preemptions(sched));
  lmsf_sched_destroy(sched);
  lmsf_cm_destroy(cm);
  return 0;
}
