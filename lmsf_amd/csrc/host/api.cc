// The C entry points of the host library (cache manager, scheduler, step metadata), for ctypes.
// Every call returns a status (0 ok, 1 cache misuse, 2 out of pages, 3 bad argument) unless it says
// otherwise; lmsf_host_last_error() gives the message of the calling thread's last failure.
#include <algorithm>
#include <cstring>
#include <string>

#include "cache_manager.h"
#include "llama_config.h"
#include "safetensors.h"
#include "scheduler.h"

using namespace lmsf;

namespace lmsf {
void llama_config_parse(const std::string& text, LmsfLlamaConfig* out);
void llama_config_validate(const LmsfLlamaConfig& c);
void rope_scaling_parse(const std::string& text, LmsfRopeScaling* out);
}  // namespace lmsf

static thread_local std::string g_error;

#define LMSF_API_BEGIN try {
#define LMSF_API_END                                   \
  }                                                    \
  catch (const Error& e) {                             \
    g_error = e.message;                               \
    return (int)e.status;                              \
  }                                                    \
  catch (const std::exception& e) {                    \
    g_error = e.what();                                \
    return (int)kValueError;                           \
  }                                                    \
  return 0;

extern "C" {

int lmsf_host_abi_version() { return 4; }
const char* lmsf_host_last_error() { return g_error.c_str(); }

// ---------------------------------------------------------------- a page pool alone

int lmsf_pool_create(int num_pages, void** out) {
  LMSF_API_BEGIN
  *out = new PagePool(num_pages);
  LMSF_API_END
}
void lmsf_pool_destroy(void* pool) { delete static_cast<PagePool*>(pool); }
int lmsf_pool_num_free(void* pool) { return static_cast<PagePool*>(pool)->num_free(); }
int lmsf_pool_allocate(void* pool, int* page) {
  LMSF_API_BEGIN
  *page = static_cast<PagePool*>(pool)->allocate();
  LMSF_API_END
}
int lmsf_pool_release(void* pool, int page) {
  LMSF_API_BEGIN
  static_cast<PagePool*>(pool)->release(page);
  LMSF_API_END
}

// ---------------------------------------------------------------- cache manager

int lmsf_cm_create(int n_groups, const int* page_size, const int* num_pages, const int* window, int num_state_slots,
                   void** out) {
  LMSF_API_BEGIN
  if (n_groups < 0 || !out) fail(kValueError, "bad arguments");
  std::vector<GroupConfig> groups;
  for (int g = 0; g < n_groups; ++g) groups.push_back(GroupConfig{page_size[g], num_pages[g], window[g]});
  *out = new CacheManager(groups, num_state_slots);
  LMSF_API_END
}
void lmsf_cm_destroy(void* cm) { delete static_cast<CacheManager*>(cm); }

int lmsf_cm_has_request(void* cm, int64_t rid) { return static_cast<CacheManager*>(cm)->has_request(rid) ? 1 : 0; }
int lmsf_cm_num_free_state_slots(void* cm) { return static_cast<CacheManager*>(cm)->num_free_state_slots(); }
int lmsf_cm_num_free_pages(void* cm, int group, int* out) {
  LMSF_API_BEGIN
  *out = static_cast<CacheManager*>(cm)->num_free_pages(group);
  LMSF_API_END
}
// info: state_slot, num_tokens, pending
int lmsf_cm_request_info(void* cm, int64_t rid, int64_t* info) {
  LMSF_API_BEGIN
  const RequestCache& rc = static_cast<CacheManager*>(cm)->request(rid);
  info[0] = rc.state_slot;
  info[1] = rc.num_tokens;
  info[2] = rc.pending;
  LMSF_API_END
}
// held[i] = tokens of rids[i] that are in the pages; 0 where known[i] is 0 or the request holds no cache.
int lmsf_cm_tokens_held(void* cm, int S, const int64_t* rids, const unsigned char* known, int64_t* held) {
  LMSF_API_BEGIN
  CacheManager* m = static_cast<CacheManager*>(cm);
  for (int i = 0; i < S; ++i) {
    held[i] = 0;
    if (known[i] && m->has_request(rids[i])) {
      held[i] = m->request(rids[i]).num_tokens;
    }
  }
  LMSF_API_END
}
// Blocks of rid in group: their number into *len, first_live into *first_live, and the pages into out if cap allows.
int lmsf_cm_block_table(void* cm, int64_t rid, int group, int* out, int cap, int* len, int* first_live) {
  LMSF_API_BEGIN
  CacheManager* m = static_cast<CacheManager*>(cm);
  m->group(group);
  const RequestCache& rc = m->request(rid);
  const std::vector<int>& t = rc.tables[group];
  *len = (int)t.size();
  if (first_live) *first_live = rc.first_live[group];
  if (out && cap >= (int)t.size() && !t.empty()) memcpy(out, t.data(), t.size() * sizeof(int));
  LMSF_API_END
}
int lmsf_cm_live_requests(void* cm, int64_t* out, int cap, int* count) {
  LMSF_API_BEGIN
  const std::vector<int64_t> live = static_cast<CacheManager*>(cm)->live_requests();
  *count = (int)live.size();
  if (out && cap >= (int)live.size() && !live.empty()) memcpy(out, live.data(), live.size() * sizeof(int64_t));
  LMSF_API_END
}
int lmsf_cm_pages_needed(void* cm, int has, int64_t rid, int64_t n_new, int* out) {
  LMSF_API_BEGIN
  static_cast<CacheManager*>(cm)->pages_needed(has != 0, rid, n_new, out);
  LMSF_API_END
}
int lmsf_cm_can_append(void* cm, int has, int64_t rid, int64_t n_new, int reserve_pages) {
  try {
    return static_cast<CacheManager*>(cm)->can_append(has != 0, rid, n_new, reserve_pages) ? 1 : 0;
  } catch (const Error& e) {
    g_error = e.message;
    return -1;
  }
}
int lmsf_cm_add_request(void* cm, int64_t rid, int* state_slot) {
  LMSF_API_BEGIN
  *state_slot = static_cast<CacheManager*>(cm)->add_request(rid).state_slot;
  LMSF_API_END
}
int lmsf_cm_append(void* cm, int64_t rid, int64_t n_new, int64_t* start) {
  LMSF_API_BEGIN
  *start = static_cast<CacheManager*>(cm)->append(rid, n_new);
  LMSF_API_END
}
int lmsf_cm_commit(void* cm, int64_t rid) {
  LMSF_API_BEGIN
  static_cast<CacheManager*>(cm)->commit(rid);
  LMSF_API_END
}
int lmsf_cm_rollback(void* cm, int64_t rid) {
  LMSF_API_BEGIN
  static_cast<CacheManager*>(cm)->rollback(rid);
  LMSF_API_END
}
int lmsf_cm_free_request(void* cm, int64_t rid) {
  LMSF_API_BEGIN
  static_cast<CacheManager*>(cm)->free_request(rid);
  LMSF_API_END
}
int lmsf_cm_reset(void* cm) {
  LMSF_API_BEGIN
  static_cast<CacheManager*>(cm)->reset();
  LMSF_API_END
}
int lmsf_cm_slot_mapping(void* cm, int64_t rid, int group, int64_t start, int64_t n, int* out) {
  LMSF_API_BEGIN
  static_cast<CacheManager*>(cm)->slot_mapping(rid, group, start, n, out);
  LMSF_API_END
}
int lmsf_cm_check_invariants(void* cm) {
  LMSF_API_BEGIN
  static_cast<CacheManager*>(cm)->check_invariants();
  LMSF_API_END
}

// A step of S entries in one call: every request that holds nothing yet is added, every entry's tokens are
// appended; starts receives the first position of each. All or nothing: on failure what was taken goes back.
int lmsf_cm_begin_step(void* cm, int S, const int64_t* rids, const int* lens, int64_t* starts, unsigned char* added) {
  CacheManager* m = static_cast<CacheManager*>(cm);
  int done = 0;
  try {
    for (; done < S; ++done) {
      added[done] = 0;
      if (!m->has_request(rids[done])) {
        m->add_request(rids[done]);
        added[done] = 1;
      }
      starts[done] = m->append(rids[done], lens[done]);
    }
    return 0;
  } catch (const Error& e) {
    g_error = e.message;
    // entry `done` failed: its append took nothing, but it may have been added
    for (int i = 0; i <= done && i < S; ++i) {
      try {
        if (i < done) m->rollback(rids[i]);
        if (added[i]) m->free_request(rids[i]);
      } catch (const Error&) {
      }
    }
    return (int)e.status;
  }
}
// The step failed after lmsf_cm_begin_step: give back what it took.
int lmsf_cm_abort_step(void* cm, int S, const int64_t* rids, const unsigned char* added) {
  LMSF_API_BEGIN
  CacheManager* m = static_cast<CacheManager*>(cm);
  for (int i = 0; i < S; ++i) {
    m->rollback(rids[i]);
    if (added[i]) m->free_request(rids[i]);
  }
  LMSF_API_END
}
int lmsf_cm_commit_step(void* cm, int S, const int64_t* rids) {
  LMSF_API_BEGIN
  CacheManager* m = static_cast<CacheManager*>(cm);
  for (int i = 0; i < S; ++i) m->commit(rids[i]);
  LMSF_API_END
}

// ---------------------------------------------------------------- step metadata

// widths[g] = the longest block table among the entries in group g (at least 1)
int lmsf_cm_step_widths(void* cm, int S, const int64_t* rids, int* widths) {
  LMSF_API_BEGIN
  CacheManager* m = static_cast<CacheManager*>(cm);
  for (int g = 0; g < m->num_groups(); ++g) widths[g] = 1;
  for (int s = 0; s < S; ++s) {
    const RequestCache& rc = m->request(rids[s]);
    for (int g = 0; g < m->num_groups(); ++g) widths[g] = std::max(widths[g], (int)rc.tables[g].size());
  }
  LMSF_API_END
}
int lmsf_step_layout(int64_t N, int64_t S, int64_t R, int G, const int* widths, int64_t* offsets, int64_t* total) {
  LMSF_API_BEGIN
  if (N < 0 || S < 0 || R < 0 || G < 0) fail(kValueError, "negative sizes");
  *total = step_layout(N, S, R, G, widths, offsets);
  LMSF_API_END
}
int lmsf_cm_fill_step(void* cm, int S, const int64_t* rids, const int64_t* starts, const int* lens, const int* widths,
                      const int64_t* offsets, int32_t* buffer) {
  LMSF_API_BEGIN
  fill_step(*static_cast<CacheManager*>(cm), S, rids, starts, lens, widths, offsets, buffer);
  LMSF_API_END
}

// ---------------------------------------------------------------- scheduler

int lmsf_sched_create(void* cm, int64_t max_num_batched_tokens, int max_num_seqs, int64_t max_model_len,
                      int64_t prefill_chunk_size, double watermark, void** out) {
  LMSF_API_BEGIN
  *out = new Scheduler(SchedulerConfig{max_num_batched_tokens, max_num_seqs, max_model_len, prefill_chunk_size, watermark},
                       static_cast<CacheManager*>(cm));
  LMSF_API_END
}
void lmsf_sched_destroy(void* s) { delete static_cast<Scheduler*>(s); }
int lmsf_sched_add(void* s, int64_t id, int64_t arrival, int64_t length) {
  LMSF_API_BEGIN
  static_cast<Scheduler*>(s)->add(id, arrival, length);
  LMSF_API_END
}
int lmsf_sched_set_progress(void* s, int n, const int64_t* ids, const int64_t* lengths, const int64_t* computed) {
  LMSF_API_BEGIN
  for (int i = 0; i < n; ++i) static_cast<Scheduler*>(s)->set_progress(ids[i], lengths[i], computed[i]);
  LMSF_API_END
}
int lmsf_sched_abort(void* s, int64_t id, int* found) {
  LMSF_API_BEGIN
  *found = static_cast<Scheduler*>(s)->abort(id) ? 1 : 0;
  LMSF_API_END
}
int lmsf_sched_finish(void* s, int64_t id) {
  LMSF_API_BEGIN
  static_cast<Scheduler*>(s)->finish(id);
  LMSF_API_END
}
// counts: scheduled, preempted, ignored, capped of the new plan
int lmsf_sched_schedule(void* s, int* counts) {
  LMSF_API_BEGIN
  const StepPlan& p = static_cast<Scheduler*>(s)->schedule();
  counts[0] = (int)p.scheduled.size();
  counts[1] = (int)p.preempted.size();
  counts[2] = (int)p.ignored.size();
  counts[3] = (int)p.capped.size();
  LMSF_API_END
}
// The last plan, into arrays of the sizes that lmsf_sched_schedule reported.
int lmsf_sched_plan(void* s, int64_t* ids, int64_t* starts, int64_t* n_tokens, int* samples, int64_t* preempted,
                    int64_t* ignored, int64_t* capped) {
  LMSF_API_BEGIN
  const StepPlan& p = static_cast<Scheduler*>(s)->plan();
  for (size_t i = 0; i < p.scheduled.size(); ++i) {
    ids[i] = p.scheduled[i].id;
    starts[i] = p.scheduled[i].start;
    n_tokens[i] = p.scheduled[i].n_tokens;
    samples[i] = p.scheduled[i].samples;
  }
  for (size_t i = 0; i < p.preempted.size(); ++i) preempted[i] = p.preempted[i];
  for (size_t i = 0; i < p.ignored.size(); ++i) ignored[i] = p.ignored[i];
  for (size_t i = 0; i < p.capped.size(); ++i) capped[i] = p.capped[i];
  LMSF_API_END
}
// which 0: waiting (front first), 1: running
int lmsf_sched_queue(void* s, int which, int64_t* out, int cap, int* count) {
  LMSF_API_BEGIN
  Scheduler* sc = static_cast<Scheduler*>(s);
  if (which == 0) {
    *count = (int)sc->waiting().size();
    if (out && cap >= *count) std::copy(sc->waiting().begin(), sc->waiting().end(), out);
  } else {
    *count = (int)sc->running().size();
    if (out && cap >= *count) std::copy(sc->running().begin(), sc->running().end(), out);
  }
  LMSF_API_END
}
int64_t lmsf_sched_num_preemptions(void* s) { return static_cast<Scheduler*>(s)->num_preemptions(); }

// ---------------------------------------------------------------- configuration

int lmsf_llama_config_parse(const char* config_json, LmsfLlamaConfig* out) {
  LMSF_API_BEGIN
  if (!config_json || !out) fail(kValueError, "bad arguments");
  llama_config_parse(config_json, out);
  LMSF_API_END
}
int lmsf_llama_config_validate(const LmsfLlamaConfig* config) {
  LMSF_API_BEGIN
  if (!config) fail(kValueError, "bad arguments");
  llama_config_validate(*config);
  LMSF_API_END
}
int lmsf_rope_scaling_parse(const char* rope_scaling_json, LmsfRopeScaling* out) {
  LMSF_API_BEGIN
  if (!rope_scaling_json || !out) fail(kValueError, "bad arguments");
  rope_scaling_parse(rope_scaling_json, out);
  LMSF_API_END
}

// ---------------------------------------------------------------- checkpoint files

// One tensor of a safetensors file. ``name`` points into the file object and lives as long as it does.
typedef struct {
  const char* name;
  char dtype[8];
  int ndim;
  int64_t shape[8];
  int64_t begin, end;   // bytes from the start of the data section
} LmsfTensorRecord;

int lmsf_safetensors_open(const char* path, void** out) {
  LMSF_API_BEGIN
  if (!path || !out) fail(kValueError, "bad arguments");
  *out = new SafetensorsFile(path);
  LMSF_API_END
}
void lmsf_safetensors_close(void* file) { delete static_cast<SafetensorsFile*>(file); }
int64_t lmsf_safetensors_count(void* file) { return (int64_t) static_cast<SafetensorsFile*>(file)->tensors().size(); }
int lmsf_safetensors_record(void* file, int64_t index, LmsfTensorRecord* out) {
  LMSF_API_BEGIN
  const auto& all = static_cast<SafetensorsFile*>(file)->tensors();
  if (!out || index < 0 || index >= (int64_t)all.size()) fail(kValueError, "bad arguments");
  const TensorRecord& r = all[(size_t)index];
  if (r.shape.size() > 8) fail(kValueError, "tensor '%s' has %zu dimensions (at most 8)", r.name.c_str(), r.shape.size());
  out->name = r.name.c_str();
  std::memset(out->dtype, 0, sizeof(out->dtype));
  std::strncpy(out->dtype, r.dtype.c_str(), sizeof(out->dtype) - 1);
  out->ndim = (int)r.shape.size();
  for (size_t i = 0; i < 8; ++i) out->shape[i] = i < r.shape.size() ? r.shape[i] : 0;
  out->begin = r.begin;
  out->end = r.end;
  LMSF_API_END
}
// Address of the data section in this process (valid until the file is closed) and its size.
const void* lmsf_safetensors_data(void* file, int64_t* size) {
  auto* f = static_cast<SafetensorsFile*>(file);
  if (size) *size = f->data_size();
  return f->data();
}

}  // extern "C"
