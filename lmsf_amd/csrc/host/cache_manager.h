// Host side of the cache: page pools, block tables and state slots. No device memory here.
//
// The reference's BlockAllocator keeps a deque of reference-counted blocks and reuses the one freed
// last (core/src/sched/block_manager.rs:14-58); BlockSpaceManager maps a sequence to its list of
// blocks (:69-347), with one pool for all layers and a model-wide sliding window that wraps the table
// (:129-135, :165-175). Here:
//  - layers with equal needs form a group with a page pool and per-request block tables of its own; a
//    group keeps every key or has a window W (a query at p reads positions > p - W only);
//  - pages go back when a request ends and, in a window group, as soon as the window has passed them;
//    the page freed last is the next one handed out, so reuse is immediate;
//  - beside the pages there are slots for per-request state of fixed size, one per live request;
//  - nothing is shared between requests: a page has one holder or none, and giving back a page that is
//    not held is an error (block_manager.rs:45-48 is the reference's double-free check).
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace lmsf {

enum Status : int { kOk = 0, kCacheError = 1, kOutOfPages = 2, kValueError = 3 };

// What the C++ side throws; the C entry points turn it into a status and a message.
struct Error {
  Status status;
  std::string message;
};
[[noreturn]] void fail(Status status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

constexpr int kReleased = -1;   // a block whose page a window has passed

class PagePool {
 public:
  explicit PagePool(int num_pages);
  int num_pages() const { return num_pages_; }
  int num_free() const { return (int)free_.size(); }
  int allocate();            // page 0 first, then LIFO
  void release(int page);
  bool is_held(int page) const { return held_[page]; }
  const std::vector<int>& free_list() const { return free_; }

 private:
  int num_pages_;
  std::vector<int> free_;
  std::vector<char> held_;
};

struct GroupConfig {
  int page_size;
  int num_pages;
  int window;   // 0: every key stays
};

struct RequestCache {
  int64_t id = 0;
  int state_slot = -1;
  int64_t num_tokens = 0;                 // tokens whose keys and values are in the pages
  int64_t pending = 0;                    // appended, not yet committed (the running step's)
  std::vector<std::vector<int>> tables;   // per group: page of logical block i, or kReleased
  std::vector<int> first_live;            // per group: first block not yet released
};

class CacheManager {
 public:
  CacheManager(const std::vector<GroupConfig>& groups, int num_state_slots);

  int num_groups() const { return (int)groups_.size(); }
  const GroupConfig& group(int g) const;
  int num_state_slots() const { return num_state_slots_; }
  bool has_request(int64_t rid) const { return requests_.count(rid) != 0; }
  const RequestCache& request(int64_t rid) const;
  const RequestCache* find(int64_t rid) const;
  std::vector<int64_t> live_requests() const;
  int num_free_pages(int g) const;
  int num_free_state_slots() const { return (int)free_slots_.size(); }

  // New pages per group that n_new more tokens of rid would take; has == false: a request that holds nothing.
  void pages_needed(bool has, int64_t rid, int64_t n_new, int* out) const;
  bool can_append(bool has, int64_t rid, int64_t n_new, int reserve_pages) const;

  const RequestCache& add_request(int64_t rid);
  int64_t append(int64_t rid, int64_t n_new);   // position of the first new token; all or nothing
  void commit(int64_t rid);                     // the appended tokens are in the pages now
  void rollback(int64_t rid);                   // undo an append that was not committed
  void free_request(int64_t rid);
  void reset();

  void slot_mapping(int64_t rid, int g, int64_t start, int64_t n, int* out) const;
  void check_invariants() const;

 private:
  RequestCache& mut(int64_t rid);
  std::vector<GroupConfig> groups_;
  std::vector<PagePool> pools_;
  int num_state_slots_;
  std::vector<int> free_slots_;
  std::unordered_map<int64_t, RequestCache> requests_;
  std::vector<int64_t> order_;   // live requests in the order they were added
};

// Offsets (int32 elements, 16-byte aligned) of the sections of a step's metadata buffer:
// token_ids[N] positions[N] seg_of[N] seg_starts[S+1] seg_first[S] state_slots[S] logit_rows[R], then per
// group slots[N] tables[S * width]. offsets has 7 + 2 G entries; returns the total.
int64_t step_layout(int64_t N, int64_t S, int64_t R, int G, const int* widths, int64_t* offsets);

// Fills every section but token_ids and logit_rows (the caller's) for S entries (request, first position,
// number of tokens). Pages that a window has passed appear as page 0 in the tables; a token whose own page
// was given back is an error.
void fill_step(const CacheManager& cm, int S, const int64_t* rids, const int64_t* starts, const int* lens,
               const int* widths, const int64_t* offsets, int32_t* buffer);

}  // namespace lmsf
