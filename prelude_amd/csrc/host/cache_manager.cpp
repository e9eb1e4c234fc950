#include "cache_manager.h"

#include <algorithm>

namespace pa {

PagePool::PagePool(int num_pages, int run) : run_(run > 1 ? run : 1), held_(num_pages > 0 ? num_pages : 0, 0) {
  const int n = capacity(), runs = (n + run_ - 1) / run_;
  claim_.assign(n, kNobody);
  stamp_.assign(n, 0);
  unclaimed_free_.assign(runs, 0);
  run_stamp_.assign(runs, 0);
  free_count_ = n;
  for (int i = 0; i < n; ++i) free_.push_back({i, 0});
  for (int r = 0; r < runs; ++r) {
    unclaimed_free_[r] = run_len(r);
    runs_.push_back({r, 0});
  }
}

// A free page becomes a held one.
void PagePool::grab(int page) {
  if (claim_[page] == kNobody) --unclaimed_free_[page / run_];
  claim_[page] = kNobody;
  held_[page] = 1;
  ++stamp_[page];   // its entry in free_ is void from now on
  --free_count_;
}

// A page that is free has lost its claim, or has just become free: its run may be whole again.
void PagePool::page_is_unclaimed_and_free(int page) {
  const int r = page / run_;
  if (++unclaimed_free_[r] == run_len(r) && run_ > 1) {
    runs_.push_back({r, ++run_stamp_[r]});
    if (runs_.size() > queue_limit(unclaimed_free_.size())) {
      std::deque<Entry> live;
      for (const Entry& e : runs_)
        if (e.stamp == run_stamp_[e.index]) live.push_back(e);
      runs_.swap(live);
    }
  }
}

// The queues are only ever popped where a hand-out falls through to them; a pool whose requests keep finding the
// page behind their last one would let void entries pile up for good.  Past twice the number of things they can
// validly hold, the void ones are dropped (the order of the others stays): constant work per page on average.
void PagePool::drop_void_entries() {
  std::deque<Entry> live;
  for (const Entry& e : free_)
    if (e.stamp == stamp_[e.index] && !held_[e.index]) live.push_back(e);
  free_.swap(live);
}

int PagePool::take(int64_t owner, int after) {
  if (free_count_ == 0) return -1;
  if (run_ > 1) {
    const int next = after + 1;
    if (after >= 0 && next < capacity() && !held_[next] && (claim_[next] == kNobody || claim_[next] == owner)) {
      grab(next);
      return next;
    }
    while (!runs_.empty()) {
      const Entry e = runs_.front();
      runs_.pop_front();
      if (e.stamp != run_stamp_[e.index] || unclaimed_free_[e.index] != run_len(e.index)) continue;
      const int first = e.index * run_;
      grab(first);
      if (owner != kNobody) {
        auto& mine = claims_of_[owner];
        for (int p = first + 1; p < first + run_len(e.index); ++p) {
          claim_[p] = owner;
          --unclaimed_free_[e.index];
          mine.push_back(p);
        }
      }
      return first;
    }
  }
  while (!free_.empty()) {
    const Entry e = free_.front();
    free_.pop_front();
    if (e.stamp != stamp_[e.index] || held_[e.index]) continue;
    grab(e.index);
    return e.index;
  }
  return -1;   // not reached while free_count_ is right
}

bool PagePool::give(int page) {
  if (!held(page)) return false;
  held_[page] = 0;
  ++free_count_;
  free_.push_back({page, ++stamp_[page]});
  if (free_.size() > queue_limit(held_.size())) drop_void_entries();
  page_is_unclaimed_and_free(page);
  return true;
}

void PagePool::release_claims(int64_t owner) {
  auto it = claims_of_.find(owner);
  if (it == claims_of_.end()) return;
  for (int p : it->second) {
    if (held_[p] || claim_[p] != owner) continue;   // taken since (by its owner or by someone in need)
    claim_[p] = kNobody;
    page_is_unclaimed_and_free(p);
  }
  claims_of_.erase(it);
}

std::string PagePool::check() const {
  int free_pages = 0;
  std::vector<int> count(unclaimed_free_.size(), 0);
  for (int p = 0; p < capacity(); ++p) {
    if (held_[p]) {
      if (claim_[p] != kNobody) return "page " + std::to_string(p) + " is held and claimed";
      continue;
    }
    ++free_pages;
    if (claim_[p] == kNobody) ++count[p / run_];
  }
  if (free_pages != free_count_) return "the count of free pages is off";
  for (size_t r = 0; r < count.size(); ++r)
    if (count[r] != unclaimed_free_[r]) return "run " + std::to_string(r) + ": the count of unclaimed free pages is off";
  if (free_.size() > queue_limit(held_.size()) || runs_.size() > queue_limit(unclaimed_free_.size()))
    return "a queue holds " + std::to_string(std::max(free_.size(), runs_.size())) + " entries, most of them void";
  // every free page can still be reached through the queue
  std::vector<uint8_t> queued(capacity(), 0);
  for (const Entry& e : free_)
    if (e.stamp == stamp_[e.index] && !held_[e.index]) queued[e.index] = 1;
  for (int p = 0; p < capacity(); ++p)
    if (!held_[p] && !queued[p]) return "free page " + std::to_string(p) + " is in no queue";
  return "";
}

CacheManager::CacheManager(int page_size, const std::vector<GroupSpec>& groups, int num_state_slots)
    : page_size_(page_size), groups_(groups), num_state_slots_(num_state_slots > 0 ? num_state_slots : 0) {
  // runs of 128 tokens: what a request is given side by side where that is free (see PagePool)
  const int run = page_size_ > 0 && page_size_ < 128 ? 128 / page_size_ : 1;
  for (const auto& g : groups_) pools_.emplace_back(g.num_pages, run);
  slot_held_.assign(num_state_slots_, 0);
  for (int i = 0; i < num_state_slots_; ++i) free_slots_.push_back(i);
}

const RequestCache* CacheManager::find(int64_t id) const {
  auto it = requests_.find(id);
  return it == requests_.end() ? nullptr : &it->second;
}

bool CacheManager::open(int64_t id, bool need_state) {
  if (requests_.count(id)) {
    error_ = "request " + std::to_string(id) + " is already live";
    return false;
  }
  RequestCache rc;
  rc.tables.resize(groups_.size());
  rc.first_live.assign(groups_.size(), 0);
  if (need_state) {
    if (free_slots_.empty()) {
      error_ = "no free state slot for request " + std::to_string(id);
      return false;
    }
    rc.state_slot = free_slots_.front();
    free_slots_.pop_front();
    slot_held_[rc.state_slot] = 1;
  }
  requests_.emplace(id, std::move(rc));
  return true;
}

int CacheManager::first_key_needed(int g, int start) const {
  const int w = groups_[g].window;
  if (w <= 0) return 0;
  return std::max(0, start - w + 1);
}

int CacheManager::pages_needed(int64_t id, int new_len, int g) const {
  const RequestCache* rc = find(id);
  const int want = table_len(new_len);
  const int have = rc ? (int)rc->tables[g].size() : 0;
  return std::max(0, want - have);
}

int CacheManager::peak_pages(int total, int chunk, int g) const {
  const int all = table_len(total);
  const int w = groups_[g].window;
  if (w <= 0) return all;
  // a portion of `chunk` tokens sees back over w - 1 keys; one more page for the misalignment at either end
  const int span = table_len(std::max(1, chunk) + w - 1) + 1;
  return std::min(all, span);
}

int CacheManager::live_pages(int64_t id, int g) const {
  const RequestCache* rc = find(id);
  if (!rc) return 0;
  int n = 0;
  for (int p : rc->tables[g]) n += p >= 0;
  return n;
}

int CacheManager::reservable_len(int64_t id) const {
  const RequestCache* rc = find(id);
  if (!rc) return 0;
  long best = -1;
  for (int g = 0; g < num_groups(); ++g) {
    const auto& table = rc->tables[g];
    const int first_key = first_key_needed(g, rc->len);
    int releasable = 0;
    for (int i = rc->first_live[g]; i < (int)table.size() && (i + 1) * page_size_ <= first_key; ++i)
      releasable += table[i] >= 0;
    const long reach = ((long)table.size() + pools_[g].free_count() + releasable) * page_size_;
    if (best < 0 || reach < best) best = reach;
  }
  if (best < 0) best = 0x7fffffff;  // no cache group at all: nothing limits the length
  return (int)std::min<long>(best, 0x7fffffff);
}

void CacheManager::release_before(RequestCache& rc, int g, int first_key) {
  auto& table = rc.tables[g];
  int& i = rc.first_live[g];
  while (i < (int)table.size() && (i + 1) * page_size_ <= first_key) {
    if (table[i] >= 0) {
      pools_[g].give(table[i]);
      table[i] = -1;
    }
    ++i;
  }
}

int CacheManager::reserve(int64_t id, int new_len) {
  auto it = requests_.find(id);
  if (it == requests_.end()) {
    error_ = "reserve: request " + std::to_string(id) + " is not live";
    return -1;
  }
  RequestCache& rc = it->second;
  if (rc.reserved_len != rc.len) {
    error_ = "reserve: request " + std::to_string(id) + " already has a portion in flight";
    return -1;
  }
  if (new_len <= rc.len) {
    error_ = "reserve: request " + std::to_string(id) + " holds " + std::to_string(rc.len) +
             " tokens, cannot extend to " + std::to_string(new_len);
    return -1;
  }
  const int G = num_groups();
  for (int g = 0; g < G; ++g) release_before(rc, g, first_key_needed(g, rc.len));
  const int want = table_len(new_len);
  for (int g = 0; g < G; ++g) {
    const int need = std::max(0, want - (int)rc.tables[g].size());
    if (need > pools_[g].free_count()) return 1;
  }
  // Every new page lies at or after the portion's first position, so it is
  // inside what the portion writes: none of them can be skipped for a window.
  for (int g = 0; g < G; ++g) {
    auto& table = rc.tables[g];
    while ((int)table.size() < want) table.push_back(pools_[g].take(id, table.empty() ? -1 : table.back()));
  }
  rc.reserved_len = new_len;
  return 0;
}

bool CacheManager::commit(int64_t id, int new_len) {
  auto it = requests_.find(id);
  if (it == requests_.end()) {
    error_ = "commit: request " + std::to_string(id) + " is not live";
    return false;
  }
  RequestCache& rc = it->second;
  if (new_len != rc.reserved_len || new_len <= rc.len) {
    error_ = "commit: request " + std::to_string(id) + " has " + std::to_string(rc.reserved_len) +
             " tokens reserved, not " + std::to_string(new_len);
    return false;
  }
  rc.len = new_len;
  rc.fresh = false;
  return true;
}

bool CacheManager::rollback(int64_t id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) {
    error_ = "rollback: request " + std::to_string(id) + " is not live";
    return false;
  }
  RequestCache& rc = it->second;
  const int keep = table_len(rc.len);
  for (int g = 0; g < num_groups(); ++g) {
    auto& table = rc.tables[g];
    while ((int)table.size() > keep) {
      if (table.back() >= 0) pools_[g].give(table.back());
      table.pop_back();
    }
    rc.first_live[g] = std::min(rc.first_live[g], (int)table.size());
  }
  rc.reserved_len = rc.len;
  return true;
}

bool CacheManager::close(int64_t id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) {
    error_ = "close: request " + std::to_string(id) + " is not live";
    return false;
  }
  RequestCache& rc = it->second;
  for (int g = 0; g < num_groups(); ++g) {
    for (int p : rc.tables[g])
      if (p >= 0) pools_[g].give(p);
    pools_[g].release_claims(id);
  }
  if (rc.state_slot >= 0) {
    slot_held_[rc.state_slot] = 0;
    free_slots_.push_back(rc.state_slot);
  }
  requests_.erase(it);
  return true;
}

bool CacheManager::fill_step(int n, const int64_t* ids, const int* starts, const int* counts, int table_stride,
                             int* positions, int* seq_of_token, int* cu_q, int* context_lens, int* state_slots,
                             int* fresh, int* block_tables, int* slots) {
  const int G = num_groups();
  int total = 0;
  for (int i = 0; i < n; ++i) total += counts[i];
  int t = 0;
  cu_q[0] = 0;
  for (int i = 0; i < n; ++i) {
    auto it = requests_.find(ids[i]);
    if (it == requests_.end()) {
      error_ = "step: request " + std::to_string(ids[i]) + " is not live";
      return false;
    }
    const RequestCache& rc = it->second;
    const int start = starts[i], end = starts[i] + counts[i];
    if (counts[i] <= 0 || start != rc.len || end != rc.reserved_len) {
      error_ = "step: request " + std::to_string(ids[i]) + " holds " + std::to_string(rc.len) + " tokens with " +
               std::to_string(rc.reserved_len) + " reserved; a portion [" + std::to_string(start) + ", " +
               std::to_string(end) + ") does not continue it";
      return false;
    }
    const int pages = table_len(end);
    if (pages > table_stride) {
      error_ = "step: block table stride " + std::to_string(table_stride) + " is smaller than " +
               std::to_string(pages) + " pages";
      return false;
    }
    for (int g = 0; g < G; ++g) {
      const auto& table = rc.tables[g];
      int* row = block_tables + ((size_t)g * n + i) * table_stride;
      for (int j = 0; j < table_stride; ++j) row[j] = j < (int)table.size() ? table[j] : -1;
      int* srow = slots + (size_t)g * total + t;
      for (int p = start; p < end; ++p) {
        const int page = table[p / page_size_];
        if (page < 0) {
          error_ = "step: request " + std::to_string(ids[i]) + " has no page for position " + std::to_string(p);
          return false;
        }
        srow[p - start] = page * page_size_ + p % page_size_;
      }
    }
    for (int p = start; p < end; ++p, ++t) {
      positions[t] = p;
      seq_of_token[t] = i;
    }
    cu_q[i + 1] = t;
    context_lens[i] = end;
    state_slots[i] = rc.state_slot;
    fresh[i] = (rc.fresh && start == 0) ? 1 : 0;
  }
  return true;
}

std::string CacheManager::audit() const {
  for (int g = 0; g < num_groups(); ++g) {
    std::vector<int> owners(pools_[g].capacity(), 0);
    for (const auto& kv : requests_) {
      for (int p : kv.second.tables[g]) {
        if (p < 0) continue;
        if (p >= pools_[g].capacity()) return "group " + std::to_string(g) + ": page id out of range";
        if (++owners[p] > 1) return "group " + std::to_string(g) + ": page " + std::to_string(p) + " is held twice";
        if (!pools_[g].held(p)) return "group " + std::to_string(g) + ": page " + std::to_string(p) + " is in a table but free";
      }
    }
    int held = 0;
    for (int p = 0; p < pools_[g].capacity(); ++p) {
      if (pools_[g].held(p)) {
        ++held;
        if (!owners[p]) return "group " + std::to_string(g) + ": page " + std::to_string(p) + " is lost (held by no request)";
      }
    }
    if (held + pools_[g].free_count() != pools_[g].capacity())
      return "group " + std::to_string(g) + ": free and held pages do not add up";
    const std::string inside = pools_[g].check();
    if (!inside.empty()) return "group " + std::to_string(g) + ": " + inside;
    for (int p = 0; p < pools_[g].capacity(); ++p) {
      const int64_t c = pools_[g].claimed_by(p);
      if (c != PagePool::kNobody && !requests_.count(c))
        return "group " + std::to_string(g) + ": page " + std::to_string(p) + " is kept for a request that is gone";
    }
  }
  std::vector<int> slot_owner(num_state_slots_, 0);
  for (const auto& kv : requests_) {
    const int s = kv.second.state_slot;
    if (s < 0) continue;
    if (s >= num_state_slots_ || !slot_held_[s]) return "state slot " + std::to_string(s) + " is used but not held";
    if (++slot_owner[s] > 1) return "state slot " + std::to_string(s) + " is held twice";
  }
  int held_slots = 0;
  for (int s = 0; s < num_state_slots_; ++s) {
    if (slot_held_[s]) {
      ++held_slots;
      if (!slot_owner[s]) return "state slot " + std::to_string(s) + " is lost";
    }
  }
  if (held_slots + (int)free_slots_.size() != num_state_slots_) return "free and held state slots do not add up";
  return "";
}

}  // namespace pa
