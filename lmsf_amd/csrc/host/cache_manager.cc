#include "cache_manager.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <unordered_set>

namespace lmsf {

void fail(Status status, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  throw Error{status, buf};
}

// ---------------------------------------------------------------- PagePool

PagePool::PagePool(int num_pages) : num_pages_(num_pages) {
  if (num_pages < 0) fail(kValueError, "num_pages must be >= 0");
  free_.reserve(num_pages);
  for (int p = num_pages - 1; p >= 0; --p) free_.push_back(p);   // page 0 is handed out first
  held_.assign(num_pages, 0);
}

int PagePool::allocate() {
  if (free_.empty()) fail(kOutOfPages, "page pool of %d pages is exhausted", num_pages_);
  const int p = free_.back();
  free_.pop_back();
  if (held_[p]) fail(kCacheError, "page %d was on the free list while held", p);
  held_[p] = 1;
  return p;
}

void PagePool::release(int page) {
  if (page < 0 || page >= num_pages_) fail(kCacheError, "page %d does not exist", page);
  if (!held_[page]) fail(kCacheError, "page %d is given back twice", page);
  held_[page] = 0;
  free_.push_back(page);
}

// ---------------------------------------------------------------- CacheManager

CacheManager::CacheManager(const std::vector<GroupConfig>& groups, int num_state_slots)
    : groups_(groups), num_state_slots_(num_state_slots) {
  if (num_state_slots < 0) fail(kValueError, "num_state_slots must be >= 0");
  for (const GroupConfig& g : groups_) {
    if (g.page_size <= 0) fail(kValueError, "page_size must be > 0");
    if (g.window < 0) fail(kValueError, "window must be > 0 or None");
    pools_.emplace_back(g.num_pages);
  }
  for (int s = num_state_slots - 1; s >= 0; --s) free_slots_.push_back(s);
}

const GroupConfig& CacheManager::group(int g) const {
  if (g < 0 || g >= num_groups()) fail(kValueError, "group %d does not exist", g);
  return groups_[g];
}

int CacheManager::num_free_pages(int g) const {
  group(g);
  return pools_[g].num_free();
}

const RequestCache* CacheManager::find(int64_t rid) const {
  auto it = requests_.find(rid);
  return it == requests_.end() ? nullptr : &it->second;
}

const RequestCache& CacheManager::request(int64_t rid) const {
  const RequestCache* rc = find(rid);
  if (!rc) fail(kCacheError, "request holds no cache");
  return *rc;
}

RequestCache& CacheManager::mut(int64_t rid) { return const_cast<RequestCache&>(request(rid)); }

std::vector<int64_t> CacheManager::live_requests() const { return order_; }

void CacheManager::pages_needed(bool has, int64_t rid, int64_t n_new, int* out) const {
  const RequestCache* rc = has ? find(rid) : nullptr;
  for (int g = 0; g < num_groups(); ++g) {
    const int64_t have = rc ? (int64_t)rc->tables[g].size() : 0;
    const int64_t total = (rc ? rc->num_tokens + rc->pending : 0) + n_new;
    const int64_t ps = groups_[g].page_size;
    const int64_t blocks = total <= 0 ? 0 : (total + ps - 1) / ps;
    out[g] = (int)std::max<int64_t>(0, blocks - have);
  }
}

bool CacheManager::can_append(bool has, int64_t rid, int64_t n_new, int reserve_pages) const {
  std::vector<int> need(num_groups());
  pages_needed(has, rid, n_new, need.data());
  if ((!has || !find(rid)) && free_slots_.empty()) return false;
  for (int g = 0; g < num_groups(); ++g)
    if (pools_[g].num_free() - need[g] < reserve_pages) return false;
  return true;
}

const RequestCache& CacheManager::add_request(int64_t rid) {
  if (has_request(rid)) fail(kCacheError, "request already holds cache");
  if (free_slots_.empty()) fail(kOutOfPages, "all %d state slots are taken", num_state_slots_);
  RequestCache rc;
  rc.id = rid;
  rc.state_slot = free_slots_.back();
  free_slots_.pop_back();
  rc.tables.resize(num_groups());
  rc.first_live.assign(num_groups(), 0);
  order_.push_back(rid);
  return requests_.emplace(rid, std::move(rc)).first->second;
}

int64_t CacheManager::append(int64_t rid, int64_t n_new) {
  if (n_new <= 0) fail(kValueError, "append needs n_new > 0");
  RequestCache& rc = mut(rid);
  if (rc.pending) fail(kCacheError, "request has an uncommitted append");
  std::vector<int> need(num_groups());
  pages_needed(true, rid, n_new, need.data());
  for (int g = 0; g < num_groups(); ++g)
    if (need[g] > pools_[g].num_free())
      fail(kOutOfPages, "request needs %d pages of group %d, %d are free", need[g], g, pools_[g].num_free());
  for (int g = 0; g < num_groups(); ++g)
    for (int i = 0; i < need[g]; ++i) rc.tables[g].push_back(pools_[g].allocate());
  rc.pending = n_new;
  return rc.num_tokens;
}

void CacheManager::commit(int64_t rid) {
  RequestCache& rc = mut(rid);
  rc.num_tokens += rc.pending;
  rc.pending = 0;
  for (int g = 0; g < num_groups(); ++g) {
    const GroupConfig& cfg = groups_[g];
    if (cfg.window == 0) continue;
    // the next query stands at position >= num_tokens and reads keys > num_tokens - window
    const int64_t first_needed = std::max<int64_t>(0, rc.num_tokens - cfg.window + 1);
    std::vector<int>& table = rc.tables[g];
    const int keep_from = (int)std::min<int64_t>(first_needed / cfg.page_size, (int64_t)table.size());
    for (int b = rc.first_live[g]; b < keep_from; ++b) {
      if (table[b] != kReleased) {
        pools_[g].release(table[b]);
        table[b] = kReleased;
      }
    }
    rc.first_live[g] = std::max(rc.first_live[g], keep_from);
  }
}

void CacheManager::rollback(int64_t rid) {
  RequestCache& rc = mut(rid);
  if (!rc.pending) return;
  rc.pending = 0;
  for (int g = 0; g < num_groups(); ++g) {
    const int64_t ps = groups_[g].page_size;
    const size_t keep = (size_t)((rc.num_tokens + ps - 1) / ps);
    std::vector<int>& table = rc.tables[g];
    while (table.size() > keep) {
      const int p = table.back();
      table.pop_back();
      if (p != kReleased) pools_[g].release(p);
    }
  }
}

void CacheManager::free_request(int64_t rid) {
  RequestCache& rc = mut(rid);
  for (int g = 0; g < num_groups(); ++g) {
    const std::vector<int>& table = rc.tables[g];
    for (auto it = table.rbegin(); it != table.rend(); ++it)
      if (*it != kReleased) pools_[g].release(*it);
  }
  free_slots_.push_back(rc.state_slot);
  requests_.erase(rid);
  order_.erase(std::find(order_.begin(), order_.end(), rid));
}

void CacheManager::reset() {
  const std::vector<int64_t> all = order_;
  for (int64_t rid : all) free_request(rid);
}

void CacheManager::slot_mapping(int64_t rid, int g, int64_t start, int64_t n, int* out) const {
  const RequestCache& rc = request(rid);
  const int64_t ps = group(g).page_size;
  const std::vector<int>& table = rc.tables[g];
  if (start < 0 || n < 0) fail(kValueError, "slot_mapping: negative range");
  for (int64_t i = 0; i < n; ++i) {
    const int64_t pos = start + i;
    if (pos / ps >= (int64_t)table.size()) fail(kCacheError, "position %ld lies beyond the request's pages", (long)pos);
    const int page = table[pos / ps];
    if (page == kReleased) fail(kCacheError, "position %ld lies in a page that was given back", (long)pos);
    out[i] = (int)(page * ps + pos % ps);
  }
}

void CacheManager::check_invariants() const {
  for (int g = 0; g < num_groups(); ++g) {
    const PagePool& pool = pools_[g];
    std::unordered_set<int> seen;
    size_t in_tables = 0;
    for (const auto& kv : requests_) {
      for (int p : kv.second.tables[g]) {
        if (p == kReleased) continue;
        ++in_tables;
        if (!seen.insert(p).second) fail(kCacheError, "group %d: a page is in two block tables", g);
        if (p < 0 || p >= pool.num_pages() || !pool.is_held(p))
          fail(kCacheError, "group %d: page %d is in a table but marked free", g, p);
      }
    }
    if ((int)in_tables + pool.num_free() != pool.num_pages())
      fail(kCacheError, "group %d: %d pages in tables + %d free != %d", g, (int)in_tables, pool.num_free(),
           pool.num_pages());
    std::unordered_set<int> free_seen(pool.free_list().begin(), pool.free_list().end());
    if (free_seen.size() != pool.free_list().size()) fail(kCacheError, "group %d: a page is on the free list twice", g);
  }
  std::unordered_set<int> slots(free_slots_.begin(), free_slots_.end());
  if (slots.size() != free_slots_.size()) fail(kCacheError, "a state slot is held twice");
  for (const auto& kv : requests_)
    if (!slots.insert(kv.second.state_slot).second) fail(kCacheError, "a state slot is held twice");
  if ((int)slots.size() != num_state_slots_) fail(kCacheError, "state slots lost");
}

// ---------------------------------------------------------------- the step's metadata

static inline int64_t align4(int64_t n) { return (n + 3) / 4 * 4; }

int64_t step_layout(int64_t N, int64_t S, int64_t R, int G, const int* widths, int64_t* offsets) {
  int64_t total = 0;
  int k = 0;
  auto section = [&](int64_t n) {
    offsets[k++] = total;
    total += align4(n);
  };
  section(N);        // token_ids
  section(N);        // positions
  section(N);        // seg_of
  section(S + 1);    // seg_starts
  section(S);        // seg_first
  section(S);        // state_slots
  section(R);        // logit_rows
  for (int g = 0; g < G; ++g) {
    section(N);                       // slots
    section(S * (int64_t)widths[g]);  // tables
  }
  return std::max<int64_t>(total, 4);
}

void fill_step(const CacheManager& cm, int S, const int64_t* rids, const int64_t* starts, const int* lens,
               const int* widths, const int64_t* offsets, int32_t* buffer) {
  const int G = cm.num_groups();
  int32_t* positions = buffer + offsets[1];
  int32_t* seg_of = buffer + offsets[2];
  int32_t* seg_starts = buffer + offsets[3];
  int32_t* seg_first = buffer + offsets[4];
  int32_t* state_slots = buffer + offsets[5];
  int64_t at = 0;
  for (int s = 0; s < S; ++s) {
    const RequestCache& rc = cm.request(rids[s]);
    if (lens[s] <= 0 || starts[s] < 0) fail(kValueError, "entry %d: bad range", s);
    seg_starts[s] = (int32_t)at;
    seg_first[s] = (int32_t)starts[s];
    state_slots[s] = rc.state_slot;
    for (int i = 0; i < lens[s]; ++i) {
      positions[at + i] = (int32_t)(starts[s] + i);
      seg_of[at + i] = s;
    }
    for (int g = 0; g < G; ++g) {
      const int64_t ps = cm.group(g).page_size;
      const std::vector<int>& table = rc.tables[g];
      const int w = widths[g];
      if ((int)table.size() > w) fail(kValueError, "entry %d: %d blocks do not fit a table of width %d", s, (int)table.size(), w);
      int32_t* slots = buffer + offsets[7 + 2 * g] + at;
      int32_t* row = buffer + offsets[8 + 2 * g] + (int64_t)s * w;
      for (int i = 0; i < lens[s]; ++i) {
        const int64_t pos = starts[s] + i;
        if (pos / ps >= (int64_t)table.size()) fail(kCacheError, "position %ld lies beyond the request's pages", (long)pos);
        const int page = table[pos / ps];
        if (page == kReleased) fail(kCacheError, "position %ld lies in a page that was given back", (long)pos);
        slots[i] = (int32_t)(page * ps + pos % ps);
      }
      for (int b = 0; b < w; ++b) row[b] = b < (int)table.size() && table[b] != kReleased ? table[b] : 0;
    }
    at += lens[s];
  }
  seg_starts[S] = (int32_t)at;
}

}  // namespace lmsf
