// Continuous batching above the step function: admits requests, cuts prompts into portions under a token
// budget, decodes, and decides what happens when pages run out.
//
// The reference's scheduler (core/src/sched/scheduler.rs:343-543) runs either a batch of whole prompts or a
// batch of decode tokens, admits a prompt only when all its blocks fit
// (core/src/sched/block_manager.rs:104-122), and on shortage preempts the latest arrival by recompute
// (:253-284, :459-490). Kept from it: first come first served by arrival, head-of-line admission with a
// watermark of free pages, preemption by recompute of the latest arrival with re-insertion at the front of
// the waiting queue, and prompts longer than the limit being ignored (:368-381). Different: a step holds
// real tokens under max_num_batched_tokens: first one token for every decoding request, then portions of
// prompts in arrival order, each at most prefill_chunk_size long.
//
// When pages run out:
//  - a new request is not admitted while its first portion does not fit above the watermark (it waits);
//  - a running request that cannot get the pages for its next tokens makes the latest-arrived running
//    request behind it that the step has not served yet give up everything it holds and go back to the front
//    of the waiting queue, to be recomputed (prompt and tokens generated so far) later;
//  - with nobody behind it, a decoding request yields in the same way itself, and a request in the middle of
//    its prompt keeps what it holds and sits the step out (the requests that do run will finish or yield);
//  - a request that is alone and still cannot continue can never continue: it is finished with reason
//    "length";
//  - a prompt that would not fit the whole pool even alone is ignored at admission (reason "length").
#pragma once
#include <cstdint>
#include <deque>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"

namespace lmsf {

// core/src/common/sequence.rs:36-64
enum SeqState : int { kWaiting = 0, kRunning = 1, kFinishedStopped = 2, kFinishedLengthCapped = 3,
                      kFinishedAborted = 4, kFinishedIgnored = 5 };

struct SchedulerConfig {      // core/src/common/config.rs:287-314
  int64_t max_num_batched_tokens;
  int max_num_seqs;
  int64_t max_model_len;
  int64_t prefill_chunk_size;   // 0: a portion is as long as the budget allows
  double watermark;             // share of pages kept free at admission (block_manager.rs:88)
};

struct SeqInfo {
  int64_t id;
  int64_t arrival;        // the FCFS order, no clocks
  int64_t length;         // prompt and generated tokens
  int64_t num_computed;   // tokens whose keys and values are in the cache
  int state;
  int64_t remaining() const { return length - num_computed; }
};

struct Scheduled {
  int64_t id;
  int64_t start;     // position of the first token of this portion
  int64_t n_tokens;
  int samples;       // the portion ends at the request's last token: a token is sampled after it
};

struct StepPlan {
  std::vector<Scheduled> scheduled;
  std::vector<int64_t> preempted;
  std::vector<int64_t> ignored;   // finished without running (too long)
  std::vector<int64_t> capped;    // finished for lack of pages while alone
};

class Scheduler {
 public:
  Scheduler(const SchedulerConfig& config, CacheManager* cache);

  void add(int64_t id, int64_t arrival, int64_t length);
  // The engine's view of a request after a step: its length and what of it is in the cache.
  void set_progress(int64_t id, int64_t length, int64_t num_computed);
  bool abort(int64_t id);       // core/src/sched/scheduler.rs:160-196: in whichever queue
  void finish(int64_t id);      // the engine decided that the request is done
  bool has_unfinished() const { return !waiting_.empty() || !running_.empty(); }
  const StepPlan& schedule();
  const StepPlan& plan() const { return plan_; }
  const std::deque<int64_t>& waiting() const { return waiting_; }
  const std::vector<int64_t>& running() const { return running_; }
  const SeqInfo* find(int64_t id) const;
  int64_t num_preemptions() const { return num_preemptions_; }

 private:
  SeqInfo& seq(int64_t id);
  void release(int64_t id);
  void forget(int64_t id) { seqs_.erase(id); }
  void preempt(int64_t id);
  void remove_running(int64_t id);
  int64_t room_tokens(const SeqInfo* s, const std::vector<int>& planned, const std::vector<int>* watermark) const;
  int64_t capacity_tokens() const;

  SchedulerConfig config_;
  CacheManager* cache_;
  std::unordered_map<int64_t, SeqInfo> seqs_;
  std::deque<int64_t> waiting_;
  std::vector<int64_t> running_;
  StepPlan plan_;
  int64_t num_preemptions_ = 0;
};

}  // namespace lmsf
