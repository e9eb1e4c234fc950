// Paged cache bookkeeping on the host: pools of pages per group of layers,
// one table of pages per request and group, release of pages a window has
// passed, and a pool of slots for per-request state of fixed size.
//
// What the reference does and where: FIFO free list and slot arithmetic,
// crates/prelude-core/src/scheduler/components/cache/block_manager.rs:12-109
// (ours hands a growing request pages that lie side by side where it can,
// and falls back to first-in first-out: see PagePool);
// slots of fixed-size state, zeroed on allocation and freed with the pages,
// crates/prelude-core/src/scheduler/components/cache/deltanet_pool.rs:54-173.
// Ours: several groups with pages of their own, windows, all-or-nothing
// reservation across groups, and the step's index arrays built here.
#pragma once
#include <algorithm>
#include <climits>
#include <cstdint>
#include <deque>
#include <string>
#include <unordered_map>
#include <vector>

namespace pa {

struct GroupSpec {
  int num_pages = 0;
  int window = 0;  // keys a layer of this group looks back over, the query's own included; 0 = all
};

// A fixed set of pages.  A page goes to whoever asks, first-in first-out, but a request's pages are kept in runs
// where that costs nothing: the attention kernels read a request's pages in order, and pages that lie side by
// side in memory stream faster than pages scattered over the pool (measured on an MI355X, 64 requests of 4,096
// keys in pages of 16: 5.7 TB/s in order, 5.6 in runs of eight pages, 5.2 scattered; a decode step of 64 requests
// whose contexts grew a page at a time in turn: 9.9 ms with runs, 10.6 without).  So a request that grows is
// given, in this order:
//   1. the page behind its last one, if that is free and no other request has a claim on it;
//   2. the first page of a whole run of `run` pages (aligned, all free, none claimed), first-in first-out among
//      such runs; the rest of the run is then claimed for it;
//   3. the page that has been free the longest, whoever claims it.
// A claim only orders the hand-out: a claimed page is free, counts as free, and is taken by anyone in step 3 when
// nothing else is left, so the pool's capacity is what it would be without claims.  Claims end when their page is
// taken or their request closes.
class PagePool {
 public:
  static constexpr int64_t kNobody = INT64_MIN;
  explicit PagePool(int num_pages, int run = 1);
  int capacity() const { return (int)held_.size(); }
  int free_count() const { return free_count_; }
  int run() const { return run_; }
  // A page for `owner`, whose last page is `after` (-1: none yet); -1 when the pool is empty.
  int take(int64_t owner = kNobody, int after = -1);
  bool give(int page);    // false when the page is not held (never double-freed silently)
  void release_claims(int64_t owner);
  bool held(int page) const { return page >= 0 && page < capacity() && held_[page]; }
  int64_t claimed_by(int page) const { return page >= 0 && page < capacity() ? claim_[page] : kNobody; }
  std::string check() const;   // "" or what is inconsistent

 private:
  struct Entry {
    int index;        // a page (in free_) or a run (in runs_)
    uint32_t stamp;   // valid while it equals the index's current stamp
  };
  int run_len(int r) const { return std::min(run_, capacity() - r * run_); }
  void grab(int page);
  void page_is_unclaimed_and_free(int page);
  void drop_void_entries();
  static size_t queue_limit(size_t things) { return 2 * things + 16; }   // entries a queue may hold, void ones included

  int run_;
  int free_count_ = 0;
  std::vector<uint8_t> held_;
  std::vector<int64_t> claim_;        // free page -> the request it is kept for, or kNobody
  std::vector<uint32_t> stamp_;       // per page: bumped when it is queued and when it is taken
  std::deque<Entry> free_;            // free pages in the order they became free (void entries are skipped)
  std::vector<int> unclaimed_free_;   // per run: pages that are free and not claimed
  std::vector<uint32_t> run_stamp_;   // per run: bumped when it is queued
  std::deque<Entry> runs_;            // runs that were whole when queued (void entries are skipped)
  std::unordered_map<int64_t, std::vector<int>> claims_of_;
};

struct RequestCache {
  int len = 0;                           // tokens whose keys and values are in the cache
  int reserved_len = 0;                  // tokens the tables cover (>= len while a step is in flight)
  std::vector<std::vector<int>> tables;  // per group: logical page -> physical page, -1 once given back
  std::vector<int> first_live;           // per group: first logical page still held
  int state_slot = -1;
  bool fresh = true;                     // no step has been committed yet
};

class CacheManager {
 public:
  CacheManager(int page_size, const std::vector<GroupSpec>& groups, int num_state_slots);

  int page_size() const { return page_size_; }
  int num_groups() const { return (int)groups_.size(); }
  const GroupSpec& group(int g) const { return groups_[g]; }
  int free_pages(int g) const { return pools_[g].free_count(); }
  int capacity_pages(int g) const { return pools_[g].capacity(); }
  int free_state_slots() const { return (int)free_slots_.size(); }
  int num_state_slots() const { return num_state_slots_; }
  int num_requests() const { return (int)requests_.size(); }
  bool has(int64_t id) const { return requests_.count(id) != 0; }
  const RequestCache* find(int64_t id) const;

  // A request enters with nothing cached.  With `need_state` it also takes a
  // state slot.  Returns false (and sets error()) if the id is live or no slot is free.
  bool open(int64_t id, bool need_state);
  // Pages of group g that extending the request from its length to new_len
  // would take from the pool (after giving back what the window has passed).
  int pages_needed(int64_t id, int new_len, int g) const;
  // Pages of group g a request of `total` tokens holds at most when it is fed
  // in portions of at most `chunk` tokens.
  int peak_pages(int total, int chunk, int g) const;
  // The largest length reserve() could extend the request to right now
  // (its own pages that a window has passed count as free).
  int reservable_len(int64_t id) const;
  // Pages of group g the request holds now.
  int live_pages(int64_t id, int g) const;
  // Make the tables cover positions [len, new_len): first gives back pages
  // that lie wholly before every key the portion can see, then takes new
  // pages in every group, all or nothing.  Returns 0, or 1 if a pool ran out
  // (nothing taken then; pages given back stay given back), or -1 on misuse.
  int reserve(int64_t id, int new_len);
  // The step that wrote [len, new_len) is done.
  bool commit(int64_t id, int new_len);
  // Drop a reservation that did not run (the step was not executed).
  bool rollback(int64_t id);
  // Everything the request holds goes back.
  bool close(int64_t id);

  // Index arrays for one step over `n` portions; entry i feeds positions
  // [start_i, start_i + count_i) of request ids[i] (reserved beforehand).
  // Row-major outputs; block tables are padded with -1 to table_stride.
  //   positions, seq_of_token : [sum count]
  //   cu_q                    : [n + 1]
  //   context_lens            : [n]            start + count
  //   state_slots, fresh      : [n]
  //   block_tables            : [groups][n][table_stride]
  //   slots                   : [groups][sum count]
  bool fill_step(int n, const int64_t* ids, const int* starts, const int* counts, int table_stride, int* positions,
                 int* seq_of_token, int* cu_q, int* context_lens, int* state_slots, int* fresh, int* block_tables,
                 int* slots);
  // Largest number of table entries any of these requests needs for new_len tokens.
  int table_len(int new_len) const { return (new_len + page_size_ - 1) / page_size_; }

  // Every page is either free or held by exactly one live request, and every
  // slot likewise.  Returns "" when consistent, else what is wrong.
  std::string audit() const;
  const std::string& error() const { return error_; }

 private:
  void release_before(RequestCache& rc, int g, int first_key_needed);
  int first_key_needed(int g, int start) const;

  int page_size_;
  std::vector<GroupSpec> groups_;
  std::vector<PagePool> pools_;
  int num_state_slots_;
  std::deque<int> free_slots_;
  std::vector<uint8_t> slot_held_;
  std::unordered_map<int64_t, RequestCache> requests_;
  std::string error_;
};

}  // namespace pa
