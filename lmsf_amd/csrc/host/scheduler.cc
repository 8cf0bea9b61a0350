#include "scheduler.h"

#include <algorithm>
#include <cmath>

namespace lmsf {

Scheduler::Scheduler(const SchedulerConfig& config, CacheManager* cache) : config_(config), cache_(cache) {
  if (config.max_num_batched_tokens <= 0 || config.max_num_seqs <= 0 || config.max_model_len <= 0)
    fail(kValueError, "scheduler limits must be > 0");
  if (config.prefill_chunk_size < 0) fail(kValueError, "prefill_chunk_size must be > 0");
  if (!cache) fail(kValueError, "scheduler needs a cache manager");
}

SeqInfo& Scheduler::seq(int64_t id) {
  auto it = seqs_.find(id);
  if (it == seqs_.end()) fail(kValueError, "the scheduler does not know this request");
  return it->second;
}

const SeqInfo* Scheduler::find(int64_t id) const {
  auto it = seqs_.find(id);
  return it == seqs_.end() ? nullptr : &it->second;
}

void Scheduler::add(int64_t id, int64_t arrival, int64_t length) {
  if (seqs_.count(id)) fail(kValueError, "request is already scheduled");
  seqs_[id] = SeqInfo{id, arrival, length, 0, kWaiting};
  waiting_.push_back(id);
}

void Scheduler::set_progress(int64_t id, int64_t length, int64_t num_computed) {
  SeqInfo& s = seq(id);
  if (num_computed < 0 || num_computed > length) fail(kValueError, "progress %ld of %ld tokens", (long)num_computed, (long)length);
  s.length = length;
  s.num_computed = num_computed;
}

void Scheduler::release(int64_t id) {
  if (cache_->has_request(id)) cache_->free_request(id);
}

void Scheduler::remove_running(int64_t id) {
  auto it = std::find(running_.begin(), running_.end(), id);
  if (it != running_.end()) running_.erase(it);
}

bool Scheduler::abort(int64_t id) {
  if (!seqs_.count(id)) return false;
  auto w = std::find(waiting_.begin(), waiting_.end(), id);
  if (w != waiting_.end()) waiting_.erase(w);
  remove_running(id);
  release(id);
  forget(id);
  return true;
}

void Scheduler::finish(int64_t id) {
  // (a request may end while it waits: one that was preempted after its last token had been sampled)
  auto w = std::find(waiting_.begin(), waiting_.end(), id);
  if (w != waiting_.end()) waiting_.erase(w);
  remove_running(id);
  release(id);
  forget(id);
}

void Scheduler::preempt(int64_t id) {
  // preemption by recompute (core/src/sched/scheduler.rs:274-284): everything the request holds goes
  // back, and it returns to the front of the waiting queue
  remove_running(id);
  release(id);
  SeqInfo& s = seq(id);
  s.num_computed = 0;
  s.state = kWaiting;
  waiting_.push_front(id);
  plan_.preempted.push_back(id);
  ++num_preemptions_;
}

int64_t Scheduler::room_tokens(const SeqInfo* s, const std::vector<int>& planned, const std::vector<int>* watermark) const {
  // how many more tokens of s (null: a new request) fit in the pages that are free now
  int64_t room = -1;
  for (int g = 0; g < cache_->num_groups(); ++g) {
    const GroupConfig& cfg = cache_->group(g);
    const int64_t free_pages = cache_->num_free_pages(g) - planned[g] - (watermark ? (*watermark)[g] : 0);
    int64_t slack = 0;
    if (s) {
      if (const RequestCache* rc = cache_->find(s->id))
        slack = (int64_t)rc->tables[g].size() * cfg.page_size - rc->num_tokens;
    }
    const int64_t r = std::max<int64_t>(0, free_pages) * cfg.page_size + slack;
    room = room < 0 ? r : std::min(room, r);
  }
  return std::max<int64_t>(room, 0);
}

int64_t Scheduler::capacity_tokens() const {
  // tokens one request could hold if it had every page of the groups that keep all keys
  int64_t cap = -1;
  for (int g = 0; g < cache_->num_groups(); ++g) {
    const GroupConfig& cfg = cache_->group(g);
    if (cfg.window != 0) continue;
    const int64_t c = (int64_t)cfg.num_pages * cfg.page_size;
    cap = cap < 0 ? c : std::min(cap, c);
  }
  return cap < 0 ? (int64_t)1 << 62 : cap;
}

const StepPlan& Scheduler::schedule() {
  plan_ = StepPlan();
  const int G = cache_->num_groups();
  int64_t budget = config_.max_num_batched_tokens;
  std::vector<int> planned(G, 0), need(G, 0), watermark(G, 0);   // planned: pages promised to earlier entries
  int planned_slots = 0;
  for (int g = 0; g < G; ++g) watermark[g] = (int)std::lrint(config_.watermark * cache_->group(g).num_pages);

  auto needed = [&](const SeqInfo* s, int64_t n) { cache_->pages_needed(s != nullptr, s ? s->id : 0, n, need.data()); };
  auto fits = [&](const SeqInfo* s, int64_t n, bool reserve) {
    needed(s, n);
    for (int g = 0; g < G; ++g)
      if (cache_->num_free_pages(g) - planned[g] - need[g] < (reserve ? watermark[g] : 0)) return false;
    return true;
  };
  auto take = [&](const SeqInfo* s, int64_t n) {
    needed(s, n);
    for (int g = 0; g < G; ++g) planned[g] += need[g];
  };
  auto chunk = [&](int64_t n) { return config_.prefill_chunk_size > 0 ? std::min(n, config_.prefill_chunk_size) : n; };

  std::stable_sort(running_.begin(), running_.end(),
                   [&](int64_t a, int64_t b) { return seqs_.at(a).arrival < seqs_.at(b).arrival; });
  // The running requests in arrival order, served in two passes: first every request that has one token to
  // run (the decoding ones; core/src/sched/scheduler.rs:459-490 is the reference's decode pass), then the
  // portions of prompts from what is left of the budget. A request that cannot get its pages makes the latest
  // arrival behind it that this step has not served yet give up its pages; if there is none it is itself the
  // one to yield.
  const std::vector<int64_t> order(running_);
  enum { kUnserved = 0, kServed = 1, kGone = 2 };
  std::vector<char> mark(order.size(), kUnserved);
  auto serve = [&](size_t i) {
    const int64_t id = order[i];
    SeqInfo& s = seq(id);
    int64_t n = s.remaining();
    if (n > 1) n = chunk(std::min(n, budget));
    while (!fits(&s, n, false)) {
      if (n > 1) {
        const int64_t room = std::min(room_tokens(&s, planned, nullptr), n - 1);   // a shorter portion may fit
        if (room >= 1) {
          n = room;
          continue;
        }
      }
      size_t victim = order.size();
      for (size_t j = order.size(); j-- > i + 1;)
        if (mark[j] == kUnserved) { victim = j; break; }
      if (victim < order.size()) {
        mark[victim] = kGone;
        preempt(order[victim]);
        continue;
      }
      bool others = !plan_.scheduled.empty();
      for (size_t j = 0; j < i && !others; ++j) others = mark[j] == kUnserved;
      if (!others) {
        // alone and still no room: it can never continue
        remove_running(id);
        s.state = kFinishedLengthCapped;
        release(id);
        plan_.capped.push_back(id);
        forget(id);
        mark[i] = kGone;
      } else if (s.remaining() == 1) {
        // a decoding request that is the latest arrival of those still unserved: it yields
        mark[i] = kGone;
        preempt(id);
      } else {
        // a prompt with nobody behind it to take pages from: it keeps what it holds and waits for the requests
        // that run in this step to finish or to yield
        mark[i] = kServed;
      }
      return;
    }
    take(&s, n);
    plan_.scheduled.push_back(Scheduled{id, s.num_computed, n, s.num_computed + n == s.length ? 1 : 0});
    budget -= n;
    mark[i] = kServed;
  };
  for (size_t i = 0; i < order.size() && budget > 0; ++i)
    if (mark[i] == kUnserved && seq(order[i]).remaining() == 1) serve(i);
  for (size_t i = 0; i < order.size() && budget > 0; ++i)
    if (mark[i] == kUnserved) serve(i);

  // admission, head of line only; nothing is admitted in a step that had to preempt
  while (!waiting_.empty() && plan_.preempted.empty() && budget > 0 && (int)running_.size() < config_.max_num_seqs) {
    const int64_t id = waiting_.front();
    SeqInfo& s = seq(id);
    const int64_t limit = std::min(config_.max_model_len, capacity_tokens());
    if (s.length > limit || s.length == 0) {
      waiting_.pop_front();
      s.state = kFinishedIgnored;
      plan_.ignored.push_back(id);
      forget(id);
      continue;
    }
    if (cache_->num_free_state_slots() - planned_slots <= 0) break;
    int64_t n = chunk(std::min(s.remaining(), budget));
    if (!fits(nullptr, n, true)) {
      const int64_t room = std::min(room_tokens(nullptr, planned, &watermark), n);
      const bool idle = running_.empty() && plan_.scheduled.empty();
      if (room < 1) {
        if (!idle) break;   // wait for pages
        // every page is free and not one token fits above the watermark: it never will
        waiting_.pop_front();
        s.state = kFinishedIgnored;
        plan_.ignored.push_back(id);
        forget(id);
        continue;
      }
      if (room < std::min<int64_t>(n, 16) && !idle) break;   // wait for pages rather than crawl
      n = room;
    }
    waiting_.pop_front();
    take(nullptr, n);
    ++planned_slots;
    s.state = kRunning;
    running_.push_back(id);
    plan_.scheduled.push_back(Scheduled{id, s.num_computed, n, s.num_computed + n == s.length ? 1 : 0});
    budget -= n;
  }
  return plan_;
}

}  // namespace lmsf
